// shape.cpp -- host-side shape / stride / broadcast algebra of the tensor-kernel library.
//
// ZeNu resolves N-d, strided and broadcast operands by recursing over the leading axis and
// issuing one 1-D kernel per row (zenu-matrix/src/with_clousers.rs:180-223).  Here the same
// legality rules are checked once, the operands are folded into one iteration space, and a
// single launch covers it.
#include <algorithm>
#include <cstdint>
#include <utility>

#include "common.hpp"

namespace zenu {

int validate_tensor(const zenu_tensor_t *t)
{
    if (!t) return ZENU_ERR_ARG;
    if (t->ndim < 0 || t->ndim > kMaxDim) return ZENU_ERR_ARG;
    for (int i = 0; i < t->ndim; i++)
        if (t->shape[i] < 0 || t->stride[i] < 0) return ZENU_ERR_ARG;
    if (!t->ptr && num_elm(*t) > 0) return ZENU_ERR_ARG;
    return ZENU_OK;
}

bool same_shape(const zenu_tensor_t &a, const zenu_tensor_t &b)
{
    if (a.ndim != b.ndim) return false;
    for (int i = 0; i < a.ndim; i++)
        if (a.shape[i] != b.shape[i]) return false;
    return true;
}

bool is_default_stride_strict(const zenu_tensor_t &t)
{
    int64_t s = 1;
    for (int i = t.ndim - 1; i >= 0; i--) {
        if (t.stride[i] != s) return false;
        s *= t.shape[i];
    }
    return true;
}

zenu_tensor_t default_view(void *ptr, int ndim, const int64_t *shape)
{
    zenu_tensor_t t;
    t.ptr = ptr;
    t.ndim = ndim;
    t.reserved = 0;
    int64_t s = 1;
    for (int i = 0; i < kMaxDim; i++) { t.shape[i] = 0; t.stride[i] = 0; }
    for (int i = ndim - 1; i >= 0; i--) {
        t.shape[i] = shape[i];
        t.stride[i] = s;
        s *= shape[i];
    }
    return t;
}

// DimDyn::is_include, dim_dyn.rs:119-130: trailing dims equal.
static bool dims_include(const zenu_tensor_t &s, const zenu_tensor_t &o)
{
    if (s.ndim < o.ndim) return dims_include(o, s);
    for (int i = 0; i < o.ndim; i++)
        if (s.shape[s.ndim - 1 - i] != o.shape[o.ndim - 1 - i]) return false;
    return true;
}

// DimDyn::is_include_bradcast, dim_dyn.rs:137-148: trailing dims equal or 1 on the other side.
static bool dims_include_broadcast(const zenu_tensor_t &s, const zenu_tensor_t &o)
{
    if (s.ndim < o.ndim) return false;
    for (int i = 0; i < o.ndim; i++) {
        int64_t od = o.shape[o.ndim - 1 - i];
        if (s.shape[s.ndim - 1 - i] == od || od == 1) continue;
        return false;
    }
    return true;
}

// larger_shape_is_x, dim_dyn.rs:24-47.  1: x larger, 0: y larger, -1: the reference panics.
static int larger_is_x(const zenu_tensor_t &x, const zenu_tensor_t &y)
{
    if (x.ndim < y.ndim) return dims_include(y, x) ? 0 : -1;
    if (x.ndim > y.ndim) return dims_include(x, y) ? 1 : -1;
    if (dims_include_broadcast(x, y)) return 1;
    if (dims_include_broadcast(y, x)) return 0;
    return -1;
}

int check_binary(const zenu_tensor_t &to, const zenu_tensor_t &lhs, const zenu_tensor_t &rhs)
{
    // array_array_array_check, with_clousers.rs:155-178
    int lx = larger_is_x(lhs, rhs);
    if (lx < 0) return ZENU_ERR_SHAPE;
    const zenu_tensor_t &larger = lx ? lhs : rhs;
    const zenu_tensor_t &smaller = lx ? rhs : lhs;
    if (!dims_include(larger, smaller)) {
        if (to.ndim < smaller.ndim) return ZENU_ERR_RANK;
        if (!dims_include_broadcast(to, smaller)) return ZENU_ERR_SHAPE;
    }
    // The reference also admits a destination shaped like the smaller operand, which its
    // recursion then walks out of bounds; only the larger shape is accepted here.
    if (!same_shape(to, larger)) return ZENU_ERR_SHAPE;
    return ZENU_OK;
}

int check_binary_assign(const zenu_tensor_t &to, const zenu_tensor_t &rhs)
{
    // array_array_check, with_clousers.rs:87-107
    if (to.ndim < rhs.ndim) return ZENU_ERR_RANK;
    if (!dims_include_broadcast(to, rhs)) return ZENU_ERR_SHAPE;
    return ZENU_OK;
}

// Matrix::broadcast, broadcast.rs:11-43, walked on shapes only: the legality test at every level of
// its recursion, the leading size-1 axes of the source it drops, and the shape equality its final
// copy_from demands.  What the reference would panic on is an error here: a source such as [1,C,1,1]
// or a column [m,1] passes the first test but fails inside the recursion.
static int broadcast_walk(const int64_t *to, int nt, const int64_t *src, int ns)
{
    zenu_tensor_t a{}, b{};
    a.ndim = nt;
    b.ndim = ns;
    for (int i = 0; i < nt; i++) a.shape[i] = to[i];
    for (int i = 0; i < ns; i++) b.shape[i] = src[i];
    if (!(dims_include(a, b) || dims_include_broadcast(a, b))) return ZENU_ERR_SHAPE;
    if (same_shape(a, b)) return ZENU_OK;
    if (ns > 0 && src[0] == 1) return broadcast_walk(to, nt, src + 1, ns - 1);
    if (nt == 0) return ZENU_ERR_RANK;
    if (to[0] == 0) return ZENU_OK;                       // no iteration of the loop over the leading axis
    if (nt - ns == 1) {                                   // copy_from(&source) on each index of the leading axis
        for (int i = 0; i < ns; i++)
            if (to[1 + i] != src[i]) return ZENU_ERR_SHAPE;
        return ZENU_OK;
    }
    return broadcast_walk(to + 1, nt - 1, src, ns);
}

int check_broadcast(const zenu_tensor_t &to, const zenu_tensor_t &source)
{
    return broadcast_walk(to.shape, to.ndim, source.shape, source.ndim);
}

// ---- operand aliasing -------------------------------------------------------------------------------
// ZeNu's ops take `&mut` outputs and `&` inputs, so an output never shares memory with an input
// except as the very same view (the *_assign forms).  Through a C ABI anything can be passed:
// operands that overlap only partly (shifted, transposed or broadcast views of the output's
// memory) would be read by some threads after others have overwritten them.  They are refused.

// [lo, hi) in bytes of everything a view can touch (strides are non-negative)
static void byte_range(const void *ptr, int ndim, const int64_t *shape, const int64_t *stride, size_t esz,
                       uintptr_t &lo, uintptr_t &hi)
{
    int64_t last = 0;
    bool empty = false;
    for (int d = 0; d < ndim; d++) {
        if (shape[d] == 0) empty = true;
        else last += (shape[d] - 1) * stride[d];
    }
    lo = reinterpret_cast<uintptr_t>(ptr);
    hi = empty ? lo : lo + (uintptr_t)(last + 1) * esz;
}

bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes)
{
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a_bytes && b_bytes && a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

bool view_overlaps(const zenu_tensor_t &t, size_t esz, const void *ptr, size_t bytes)
{
    uintptr_t lo, hi;
    byte_range(t.ptr, t.ndim, t.shape, t.stride, esz, lo, hi);
    return ranges_overlap(reinterpret_cast<const void *>(lo), (size_t)(hi - lo), ptr, bytes);
}

int check_output_alias(const zenu_tensor_t &out, const zenu_tensor_t &in, size_t esz)
{
    uintptr_t o0, o1, i0, i1;
    byte_range(out.ptr, out.ndim, out.shape, out.stride, esz, o0, o1);
    byte_range(in.ptr, in.ndim, in.shape, in.stride, esz, i0, i1);
    if (o0 >= i1 || i0 >= o1 || o0 == o1 || i0 == i1) return ZENU_OK;
    if (out.ptr != in.ptr || out.ndim != in.ndim) return ZENU_ERR_ARG;
    for (int d = 0; d < out.ndim; d++) {
        if (out.shape[d] != in.shape[d]) return ZENU_ERR_ARG;
        if (out.shape[d] > 1 && out.stride[d] != in.stride[d]) return ZENU_ERR_ARG;
    }
    return ZENU_OK;
}

int ew_check_alias(const EwProblem &p, size_t esz)
{
    uintptr_t o0, o1;
    byte_range(p.ptr[0], p.ndim, p.shape, p.stride[0], esz, o0, o1);
    if (o0 == o1) return ZENU_OK;
    for (int o = 1; o < p.nops; o++) {
        uintptr_t i0, i1;
        byte_range(p.ptr[o], p.ndim, p.shape, p.stride[o], esz, i0, i1);
        if (o0 >= i1 || i0 >= o1) continue;
        // overlapping: only the output's own view is allowed (same start, same stride on every dim)
        if (p.ptr[o] != p.ptr[0]) return ZENU_ERR_ARG;
        for (int d = 0; d < p.ndim; d++)
            if (p.shape[d] > 1 && p.stride[o][d] != p.stride[0][d]) return ZENU_ERR_ARG;
    }
    return ZENU_OK;
}

void ew_set_operand(EwProblem &p, int slot, const zenu_tensor_t &t, int out_ndim,
                    const int64_t *out_shape)
{
    p.ptr[slot] = t.ptr;
    int lead = out_ndim - t.ndim;
    for (int d = 0; d < out_ndim; d++) {
        int td = d - lead;
        if (td < 0) {
            p.stride[slot][d] = 0;  // missing leading dim: get_tmp_matrix passes it through
        } else if (t.shape[td] == 1 && out_shape[d] != 1) {
            p.stride[slot][d] = 0;  // size-1 dim: index 0 every time (with_clousers.rs:16-17)
        } else {
            p.stride[slot][d] = t.stride[td];
        }
    }
}

void ew_collapse(EwProblem &p)
{
    p.numel = 1;
    for (int d = 0; d < p.ndim; d++) p.numel *= p.shape[d];

    // 1. drop size-1 dims
    int nd = 0;
    for (int d = 0; d < p.ndim; d++) {
        if (p.shape[d] == 1) continue;
        p.shape[nd] = p.shape[d];
        for (int o = 0; o < p.nops; o++) p.stride[o][nd] = p.stride[o][d];
        nd++;
    }
    p.ndim = nd;
    if (nd == 0) return;

    // 2. order dims by decreasing output stride (stable), so the output is written as
    //    sequentially as its layout allows.  Elementwise work is order independent.
    int order[kMaxDim];
    for (int d = 0; d < nd; d++) order[d] = d;
    std::stable_sort(order, order + nd,
                     [&](int a, int b) { return p.stride[0][a] > p.stride[0][b]; });
    EwProblem q = p;
    for (int d = 0; d < nd; d++) {
        p.shape[d] = q.shape[order[d]];
        for (int o = 0; o < p.nops; o++) p.stride[o][d] = q.stride[o][order[d]];
    }

    // 3. merge dim d+1 into d when stride[d] == stride[d+1]*shape[d+1] for every operand
    int w = 0;
    for (int d = 1; d < nd; d++) {
        bool mergeable = true;
        for (int o = 0; o < p.nops; o++)
            if (p.stride[o][w] != p.stride[o][d] * p.shape[d]) { mergeable = false; break; }
        if (mergeable) {
            p.shape[w] *= p.shape[d];
            for (int o = 0; o < p.nops; o++) p.stride[o][w] = p.stride[o][d];
        } else {
            w++;
            p.shape[w] = p.shape[d];
            for (int o = 0; o < p.nops; o++) p.stride[o][w] = p.stride[o][d];
        }
    }
    p.ndim = w + 1;
}

}  // namespace zenu
