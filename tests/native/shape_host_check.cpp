// Host-only check of the shape / stride algebra in zenu_amd/csrc/shape.cpp (no GPU): seeded random
// elementwise problems -- up to six dims, three operands, permuted, sliced and broadcast strides --
// go through ew_set_operand + ew_collapse, and the collapsed problem must visit exactly the
// (output offset, input offsets) tuples of the original one; the alias rules are compared with an
// element-by-element model of the views.  Prints "ok <name>" per group; exit status 0 when all hold.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <set>
#include <tuple>
#include <vector>

#include "../../zenu_amd/csrc/shape.cpp"

using namespace zenu;
typedef std::tuple<int64_t, int64_t, int64_t> Triple;

static std::vector<Triple> enumerate(const EwProblem &p)
{
    std::vector<Triple> out;
    int64_t idx[kMaxDim] = {0, 0, 0, 0, 0, 0};
    int64_t n = 1;
    for (int d = 0; d < p.ndim; d++) n *= p.shape[d];
    for (int64_t i = 0; i < n; i++) {
        int64_t off[3] = {0, 0, 0};
        for (int d = 0; d < p.ndim; d++)
            for (int o = 0; o < p.nops; o++) off[o] += idx[d] * p.stride[o][d];
        out.emplace_back(off[0], off[1], off[2]);
        for (int d = p.ndim - 1; d >= 0; d--) {
            if (++idx[d] < p.shape[d]) break;
            idx[d] = 0;
        }
    }
    return out;
}

// a random view of `shape` inside a fresh base: permuted base layout, a step and an offset per dim
static zenu_tensor_t random_view(std::mt19937 &r, int nd, const int64_t *shape, float *base)
{
    zenu_tensor_t t = {};
    t.ndim = nd;
    int perm[kMaxDim];
    for (int d = 0; d < nd; d++) perm[d] = d;
    std::shuffle(perm, perm + nd, r);
    int64_t run = 1, off = 0;
    for (int k = nd - 1; k >= 0; k--) {          // perm[k] is the k-th slowest dim of the base
        const int d = perm[k];
        const int64_t step = 1 + (int64_t)(r() % 3), lead = (int64_t)(r() % 2);
        t.shape[d] = shape[d];
        t.stride[d] = run * step;
        off += lead * run;
        run *= shape[d] * step + lead + 1;
    }
    t.ptr = base + off;
    return t;
}

static int check_collapse(unsigned seed)
{
    std::mt19937 r(seed);
    static float base[3][1];                      // only addresses are used, nothing is dereferenced
    for (int rep = 0; rep < 4000; rep++) {
        const int nd = (int)(r() % 7);
        int64_t shape[kMaxDim];
        int64_t total = 1;
        for (int d = 0; d < nd; d++) {
            shape[d] = 1 + (int64_t)(r() % 5);
            total *= shape[d];
        }
        zenu_tensor_t to = random_view(r, nd, shape, base[0]);
        EwProblem p;
        p.nops = 3;
        p.ndim = nd;
        for (int d = 0; d < nd; d++) p.shape[d] = shape[d];
        for (int d = nd; d < kMaxDim; d++) p.shape[d] = 1;
        for (int o = 0; o < kMaxOperands; o++) {
            p.ptr[o] = nullptr;
            for (int d = 0; d < kMaxDim; d++) p.stride[o][d] = 0;
        }
        p.ptr[0] = to.ptr;
        for (int d = 0; d < nd; d++) p.stride[0][d] = to.stride[d];
        for (int o = 1; o < 3; o++) {
            // an input: the output's rank with some dims 1, or fewer (trailing) dims
            int ind = nd;
            int64_t ishape[kMaxDim];
            if (nd && r() % 2) ind = (int)(r() % (nd + 1));
            for (int d = 0; d < ind; d++) {
                const int64_t full = shape[nd - ind + d];
                ishape[d] = (r() % 3 == 0) ? 1 : full;
            }
            zenu_tensor_t in = random_view(r, ind, ishape, base[o]);
            ew_set_operand(p, o, in, nd, shape);
        }
        std::vector<Triple> before = enumerate(p);
        EwProblem q = p;
        ew_collapse(q);
        if (q.numel != total) { std::printf("numel %lld != %lld\n", (long long)q.numel, (long long)total); return 1; }
        if (q.ndim > nd || q.ndim < 0) { std::printf("rank grew\n"); return 1; }
        for (int d = 0; d < q.ndim; d++)
            if (q.shape[d] <= 1) { std::printf("a dim of size %lld survived\n", (long long)q.shape[d]); return 1; }
        std::vector<Triple> after = enumerate(q);
        std::sort(before.begin(), before.end());
        std::sort(after.begin(), after.end());
        if (before != after) { std::printf("seed %u rep %d: the collapsed problem visits other offsets\n", seed, rep); return 1; }
        // the output's strides never increase from one collapsed dim to the next
        for (int d = 1; d < q.ndim; d++)
            if (q.stride[0][d] > q.stride[0][d - 1]) { std::printf("output dims out of order\n"); return 1; }
    }
    return 0;
}

static std::set<const float *> elements(const zenu_tensor_t &t)
{
    std::set<const float *> s;
    int64_t idx[kMaxDim] = {0, 0, 0, 0, 0, 0};
    int64_t n = num_elm(t);
    for (int64_t i = 0; i < n; i++) {
        int64_t off = 0;
        for (int d = 0; d < t.ndim; d++) off += idx[d] * t.stride[d];
        s.insert(static_cast<const float *>(t.ptr) + off);
        for (int d = t.ndim - 1; d >= 0; d--) {
            if (++idx[d] < t.shape[d]) break;
            idx[d] = 0;
        }
    }
    return s;
}

static int check_alias(unsigned seed)
{
    std::mt19937 r(seed);
    static float arena[4096];
    int refused = 0, accepted = 0;
    for (int rep = 0; rep < 20000; rep++) {
        const int nd = 1 + (int)(r() % 3);
        int64_t shape[kMaxDim];
        for (int d = 0; d < nd; d++) shape[d] = 1 + (int64_t)(r() % 4);
        zenu_tensor_t out = random_view(r, nd, shape, arena + r() % 64);
        zenu_tensor_t in = (r() % 4 == 0) ? out : random_view(r, nd, shape, arena + r() % 64);
        if (r() % 8 == 0) in.ptr = out.ptr;
        const int rc = check_output_alias(out, in, sizeof(float));
        const std::set<const float *> eo = elements(out), ei = elements(in);
        bool share = false;
        for (const float *e : ei) share = share || eo.count(e);
        bool same_view = in.ptr == out.ptr;
        for (int d = 0; d < nd; d++) same_view = same_view && (shape[d] == 1 || in.stride[d] == out.stride[d]);
        if (share && !same_view && rc == ZENU_OK) { std::printf("seed %u rep %d: shared elements were accepted\n", seed, rep); return 1; }
        if (same_view && rc != ZENU_OK) { std::printf("seed %u rep %d: the output's own view was refused\n", seed, rep); return 1; }
        const float *olo = *eo.begin(), *ohi = *eo.rbegin(), *ilo = *ei.begin(), *ihi = *ei.rbegin();
        if ((ohi < ilo || ihi < olo) && rc != ZENU_OK) { std::printf("seed %u rep %d: disjoint ranges were refused\n", seed, rep); return 1; }
        (rc == ZENU_OK ? accepted : refused)++;
    }
    if (refused < 1000 || accepted < 1000) { std::printf("the cases are one-sided: %d refused, %d accepted\n", refused, accepted); return 1; }
    return 0;
}

static int check_rules()
{
    // check_binary / check_broadcast on the shapes of the reference's own tests (dim_dyn.rs:24-58,
    // broadcast.rs:13-44): the larger operand's shape wins, trailing dims must match or be 1
    auto T = [](std::initializer_list<int64_t> s) {
        zenu_tensor_t t = {};
        static float x;
        t.ptr = &x;
        t.ndim = (int)s.size();
        int d = 0;
        for (int64_t v : s) t.shape[d++] = v;
        int64_t run = 1;
        for (int k = t.ndim - 1; k >= 0; k--) { t.stride[k] = run; run *= t.shape[k]; }
        return t;
    };
    if (check_binary(T({2, 3}), T({2, 3}), T({3})) != ZENU_OK) return 1;
    if (check_binary(T({2, 3}), T({3}), T({2, 3})) != ZENU_OK) return 1;
    if (check_binary(T({2, 3}), T({2, 3}), T({2, 1})) != ZENU_OK) return 1;
    if (check_binary(T({2, 3}), T({2, 3}), T({2})) == ZENU_OK) return 1;        // [2] against [2,3]: trailing dims differ
    if (check_binary(T({3, 2}), T({2, 3}), T({3})) == ZENU_OK) return 1;        // destination of another shape
    if (check_binary(T({4, 2, 3}), T({4, 2, 3}), T({2, 3})) != ZENU_OK) return 1;
    if (check_broadcast(T({4, 2, 3}), T({2, 3})) != ZENU_OK) return 1;
    if (check_broadcast(T({4, 2, 3}), T({1, 3})) != ZENU_OK) return 1;
    if (check_broadcast(T({4, 2, 3}), T({4, 2})) == ZENU_OK) return 1;
    zenu_tensor_t bad = T({2, 3});
    bad.stride[0] = -3;
    if (validate_tensor(&bad) != ZENU_ERR_ARG) return 1;
    bad = T({2, 3});
    bad.ndim = 7;
    if (validate_tensor(&bad) != ZENU_ERR_ARG) return 1;
    if (validate_tensor(nullptr) != ZENU_ERR_ARG) return 1;
    return 0;
}

int main()
{
    int rc = 0;
    for (unsigned seed = 1; seed <= 5; seed++) rc |= check_collapse(seed);
    if (!rc) std::printf("ok collapse\n");
    int ra = 0;
    for (unsigned seed = 11; seed <= 13; seed++) ra |= check_alias(seed);
    if (!ra) std::printf("ok alias\n");
    const int rr = check_rules();
    if (!rr) std::printf("ok rules\n");
    return rc | ra | rr;
}
