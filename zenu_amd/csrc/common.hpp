// common.hpp -- shared declarations of the gfx950 tensor-kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/zenu_hip.h"

namespace zenu {

// ---- error plumbing -------------------------------------------------------------------------
void set_last_hip_error(hipError_t e);

#define ZENU_HIP_TRY(expr)                       \
    do {                                         \
        hipError_t _e = (expr);                  \
        if (_e != hipSuccess) {                  \
            ::zenu::set_last_hip_error(_e);      \
            return ZENU_ERR_HIP;                 \
        }                                        \
    } while (0)

// After a kernel launch: pick up launch-configuration errors without synchronising.
#define ZENU_LAUNCH_CHECK() ZENU_HIP_TRY(hipGetLastError())

inline hipStream_t as_stream(zenu_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// ---- temporary device workspace from the caching allocator (stream ordered) ------------------
struct Workspace {
    void *ptr = nullptr;
    hipStream_t stream = nullptr;
    int status = ZENU_OK;
    Workspace(size_t bytes, hipStream_t s);
    ~Workspace();
    Workspace(const Workspace &) = delete;
    Workspace &operator=(const Workspace &) = delete;
};

// ---- shape algebra (host) ---------------------------------------------------------------------
constexpr int kMaxDim = ZENU_MAX_DIM;
constexpr int kMaxOperands = 3;  // out + up to two inputs

struct Dims {
    int ndim = 0;
    int64_t shape[kMaxDim] = {0, 0, 0, 0, 0, 0};
};

inline int64_t num_elm(const zenu_tensor_t &t)
{
    int64_t n = 1;
    for (int i = 0; i < t.ndim; i++) n *= t.shape[i];
    return n;
}

int validate_tensor(const zenu_tensor_t *t);  // ZENU_OK or ZENU_ERR_ARG
bool same_shape(const zenu_tensor_t &a, const zenu_tensor_t &b);
bool is_default_stride_strict(const zenu_tensor_t &t);
// a row-major (default stride, dim/mod.rs:70-92) view of `ptr` with the given shape
zenu_tensor_t default_view(void *ptr, int ndim, const int64_t *shape);

// Broadcasting legality, restated from zenu-matrix/src/dim/dim_dyn.rs:24-58,119-148 and
// zenu-matrix/src/with_clousers.rs:87-107,155-178.
int check_binary(const zenu_tensor_t &to, const zenu_tensor_t &lhs, const zenu_tensor_t &rhs);
int check_binary_assign(const zenu_tensor_t &to, const zenu_tensor_t &rhs);
int check_broadcast(const zenu_tensor_t &to, const zenu_tensor_t &source);

// An elementwise problem over `nops` operands (operand 0 is the output) sharing one iteration
// space.  Input strides are already broadcast-expanded (0 on broadcast dims) and aligned to the
// output's rank.  collapse() drops size-1 dims, orders dims by decreasing output stride and merges
// neighbours that are jointly contiguous in every operand.
struct EwProblem {
    int nops = 0;
    int ndim = 0;
    int64_t shape[kMaxDim];
    int64_t stride[kMaxOperands][kMaxDim];
    void *ptr[kMaxOperands];
    int64_t numel = 0;
};

// Right-align `t` against the output rank with ZeNu's rule (a dim of 1, or a missing leading
// dim, broadcasts) and store it as operand `slot`.
void ew_set_operand(EwProblem &p, int slot, const zenu_tensor_t &t, int out_ndim,
                    const int64_t *out_shape);
void ew_collapse(EwProblem &p);
// ZENU_ERR_ARG when an input shares memory with the output other than as the output's own view
int ew_check_alias(const EwProblem &p, size_t esz);
int check_output_alias(const zenu_tensor_t &out, const zenu_tensor_t &in, size_t esz);
bool ranges_overlap(const void *a, size_t a_bytes, const void *b, size_t b_bytes);
bool view_overlaps(const zenu_tensor_t &t, size_t esz, const void *ptr, size_t bytes);

// ---- device properties cached at init ---------------------------------------------------------
struct DeviceInfo {
    int device = 0;
    int num_cus = 256;
    size_t lds_per_block = 65536;
};
const DeviceInfo &device_info();
int ensure_init();

}  // namespace zenu
