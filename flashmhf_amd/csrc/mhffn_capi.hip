// C ABI of libmhffn_hip.so: argument validation, error codes, dispatch.  No torch, no pybind, no allocation.
#include "../../include/mhffn.h"
#include "mhffn_common.hpp"

// Scratch of mhffn_bwd_static: device memory that belongs to this code object, so the call needs no allocation.  Every
// GPU the library is loaded on holds its own copy at its own address until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress; kernels get the address that call returned, never the name.
static __device__ __align__(256) unsigned char scratch[MHFFN_STATIC_SCRATCH_BYTES];

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_dims_impl(const mhffn_dims* d, int dtype)
{
    if (!d) return MHFFN_ERR_NULL_POINTER;
    if (dtype != MHFFN_DTYPE_BF16 && dtype != MHFFN_DTYPE_F32) return MHFFN_ERR_DTYPE;
    if (d->B <= 0 || d->H <= 0 || d->Hkuv <= 0 || d->S <= 0 || d->E <= 0 || d->d_e <= 0 || d->d_h <= 0)
        return MHFFN_ERR_SHAPE;
    if (d->H % d->Hkuv != 0) return MHFFN_ERR_SHAPE;
    if (dtype == MHFFN_DTYPE_F32) {           // fp32 correctness path: generic tiles, no MFMA
        if (d->d_h % 8 != 0 || d->d_h > 128) return MHFFN_ERR_HEAD_DIM;
    } else {
        if (d->d_h != 64 && d->d_h != 96 && d->d_h != 128) return MHFFN_ERR_HEAD_DIM;
        if (d->d_e % 32 != 0) return MHFFN_ERR_EXPERT_DIM;
    }
    // index arithmetic inside the kernels is 64-bit for rows, 32-bit for per-(b,h) token indices and grid extents
    if ((long long)d->B > 65535 || (long long)d->S > (1ll << 30)) return MHFFN_ERR_SHAPE;
    if ((long long)d->B * d->H * d->S >= (1ll << 31)) return MHFFN_ERR_SHAPE;   // token rows are counted in 32 bits
    return MHFFN_OK;
}

mhffn::Dims to_dims(const mhffn_dims* d, int token_layout = 0)
{
    return mhffn::Dims{d->B, d->H, d->Hkuv, d->S, d->d_h, d->E, d->d_e, token_layout};
}

std::atomic<void*> scratch_addr[mhffn::LDS_OPTIN_MAX_DEVICES];   // per device, looked up on the first call there

hipError_t static_scratch_of_current_device(void** out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= mhffn::LDS_OPTIN_MAX_DEVICES) return hipErrorInvalidDevice;
    void* p = scratch_addr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        scratch_addr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return hipSuccess;
}

}  // namespace

extern "C" {

const char* mhffn_strerror(int code)
{
    switch (code) {
        case MHFFN_OK: return "ok";
        case MHFFN_ERR_NULL_POINTER: return "null pointer argument";
        case MHFFN_ERR_DTYPE: return "unsupported dtype (Q, K, U, V must all be bfloat16 or all float32; R float32)";
        case MHFFN_ERR_HEAD_DIM: return "unsupported head dim (bf16: d_h must be 64, 96 or 128; fp32: a multiple of 8 up to 128)";
        case MHFFN_ERR_EXPERT_DIM: return "unsupported expert dim (bf16: d_e must be a multiple of 32)";
        case MHFFN_ERR_SHAPE:
            return "invalid extents (all must be positive, H a multiple of Hkuv; gate kernels: E <= 64), token layout or phase mask";
        case MHFFN_ERR_WORKSPACE: return "workspace missing or too small";
        case MHFFN_ERR_LAUNCH: return "kernel launch failed";
        case MHFFN_ERR_ALIGNMENT: return "pointer not 16-byte aligned";
        case MHFFN_ERR_STATIC_SCRATCH:
            return "problem too large for mhffn_bwd_static's fixed scratch (MHFFN_STATIC_SCRATCH_BYTES); use mhffn_bwd";
    }
    return "unknown error code";
}

int mhffn_is_supported(int d_h, int d_e, int dtype)
{
    if (dtype == MHFFN_DTYPE_F32) return d_h > 0 && d_h % 8 == 0 && d_h <= 128 && d_e > 0;
    if (dtype != MHFFN_DTYPE_BF16) return 0;
    return (d_h == 64 || d_h == 96 || d_h == 128) && d_e > 0 && d_e % 32 == 0;
}

int mhffn_check_dims(const mhffn_dims* dims, int dtype) { return check_dims_impl(dims, dtype); }

size_t mhffn_fwd_workspace_bytes(const mhffn_dims* dims, int dtype)
{
    if (check_dims_impl(dims, dtype) != MHFFN_OK) return 0;
    if (dtype == MHFFN_DTYPE_F32) return 0;
    return mhffn::fwd_workspace_bytes_bf16(to_dims(dims));
}

size_t mhffn_bwd_workspace_bytes(const mhffn_dims* dims, int dtype)
{
    if (check_dims_impl(dims, dtype) != MHFFN_OK) return 0;
    if (dtype == MHFFN_DTYPE_F32) return mhffn::bwd_workspace_bytes_f32(to_dims(dims));
    return mhffn::bwd_workspace_bytes_bf16(to_dims(dims));
}

int mhffn_fwd_layout(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                     void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, int token_layout,
                     void* stream, int phases)
{
    const int rc = check_dims_impl(dims, dtype);
    if (rc != MHFFN_OK) return rc;
    if (token_layout != MHFFN_TOKENS_BHSD && token_layout != MHFFN_TOKENS_BSHD) return MHFFN_ERR_SHAPE;
    if (phases & ~MHFFN_FWD_ALL) return MHFFN_ERR_SHAPE;       // a bit this build does not define: refuse, do not ignore
    if (!Q || !K || !U || !V || !R || !O) return MHFFN_ERR_NULL_POINTER;
    if (!aligned16(Q) || !aligned16(K) || !aligned16(U) || !aligned16(V) || !aligned16(R) || !aligned16(O) ||
        !aligned16(workspace))
        return MHFFN_ERR_ALIGNMENT;
    const mhffn::Dims d = to_dims(dims, token_layout);
    if (dtype == MHFFN_DTYPE_F32) {
        if (!(phases & MHFFN_FWD_MAIN)) return MHFFN_OK;
        return mhffn::launch_fwd_f32(Q, K, U, V, R, O, d, (hipStream_t)stream) == hipSuccess ? MHFFN_OK : MHFFN_ERR_LAUNCH;
    }
    const size_t need = mhffn::fwd_workspace_bytes_bf16(d);
    if (need > 0 && (!workspace || workspace_bytes < need)) return MHFFN_ERR_WORKSPACE;
    const hipError_t err = mhffn::launch_fwd_bf16(Q, K, U, V, R, O, workspace, d, (hipStream_t)stream, phases);
    return err == hipSuccess ? MHFFN_OK : MHFFN_ERR_LAUNCH;
}

int mhffn_fwd_phases(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
                     void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, void* stream,
                     int phases)
{
    return mhffn_fwd_layout(Q, K, U, V, R, O, workspace, workspace_bytes, dims, dtype, MHFFN_TOKENS_BHSD, stream, phases);
}

int mhffn_fwd(const void* Q, const void* K, const void* U, const void* V, const float* R, void* O,
              void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, void* stream)
{
    return mhffn_fwd_phases(Q, K, U, V, R, O, workspace, workspace_bytes, dims, dtype, stream, MHFFN_FWD_ALL);
}

int mhffn_bwd_layout(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_dtype,
                     void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, int token_layout,
                     void* stream, int phases)
{
    const int rc = check_dims_impl(dims, dtype);
    if (rc != MHFFN_OK) return rc;
    if (token_layout != MHFFN_TOKENS_BHSD && token_layout != MHFFN_TOKENS_BSHD) return MHFFN_ERR_SHAPE;
    if (grad_w_dtype != MHFFN_DTYPE_BF16 && grad_w_dtype != MHFFN_DTYPE_F32) return MHFFN_ERR_DTYPE;
    if (phases & ~MHFFN_BWD_ALL) return MHFFN_ERR_SHAPE;       // a bit this build does not define: refuse, do not ignore
    if (!Q || !K || !U || !V || !R || !dO || !dQ || !dK || !dU || !dV || !dR) return MHFFN_ERR_NULL_POINTER;
    const void* ptrs[] = {Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, workspace};
    for (const void* p : ptrs)
        if (!aligned16(p)) return MHFFN_ERR_ALIGNMENT;
    const mhffn::Dims d = to_dims(dims, token_layout);
    const size_t need = dtype == MHFFN_DTYPE_F32 ? mhffn::bwd_workspace_bytes_f32(d) : mhffn::bwd_workspace_bytes_bf16(d);
    if (need > 0 && (!workspace || workspace_bytes < need)) return MHFFN_ERR_WORKSPACE;
    if (dtype == MHFFN_DTYPE_F32)
        return mhffn::launch_bwd_f32(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_dtype == MHFFN_DTYPE_F32, workspace, d,
                                     (hipStream_t)stream, phases) == hipSuccess
                   ? MHFFN_OK
                   : MHFFN_ERR_LAUNCH;
    const hipError_t err = mhffn::launch_bwd_bf16(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR,
                                                  grad_w_dtype == MHFFN_DTYPE_F32, workspace, need, d,
                                                  (hipStream_t)stream, phases);
    return err == hipSuccess ? MHFFN_OK : MHFFN_ERR_LAUNCH;
}

int mhffn_bwd_static(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_dtype,
                     const mhffn_dims* dims, int dtype, int token_layout, void* stream)
{
    const int rc = check_dims_impl(dims, dtype);
    if (rc != MHFFN_OK) return rc;
    if (token_layout != MHFFN_TOKENS_BHSD && token_layout != MHFFN_TOKENS_BSHD) return MHFFN_ERR_SHAPE;
    if (grad_w_dtype != MHFFN_DTYPE_BF16 && grad_w_dtype != MHFFN_DTYPE_F32) return MHFFN_ERR_DTYPE;
    if (!Q || !K || !U || !V || !R || !dO || !dQ || !dK || !dU || !dV || !dR) return MHFFN_ERR_NULL_POINTER;
    const void* ptrs[] = {Q, K, U, V, R, dO, dQ, dK, dU, dV, dR};
    for (const void* p : ptrs)
        if (!aligned16(p)) return MHFFN_ERR_ALIGNMENT;
    const mhffn::Dims d = to_dims(dims, token_layout);
    // The float32 kernels take exactly the workspace they ask for.  The bfloat16 launch runs with as many token slices
    // as the array holds partial sums for (with one slice it needs none), so it never exceeds the array.
    const size_t need = dtype == MHFFN_DTYPE_F32 ? mhffn::bwd_workspace_bytes_f32(d) : 0;
    if (need > MHFFN_STATIC_SCRATCH_BYTES) return MHFFN_ERR_STATIC_SCRATCH;
    void* ws = nullptr;
    if (static_scratch_of_current_device(&ws) != hipSuccess) return MHFFN_ERR_LAUNCH;
    hipError_t err;
    if (dtype == MHFFN_DTYPE_F32)
        err = mhffn::launch_bwd_f32(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_dtype == MHFFN_DTYPE_F32, ws, d,
                                    (hipStream_t)stream, MHFFN_BWD_ALL);
    else
        err = mhffn::launch_bwd_bf16(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_dtype == MHFFN_DTYPE_F32, ws,
                                     (size_t)MHFFN_STATIC_SCRATCH_BYTES, d, (hipStream_t)stream, MHFFN_BWD_ALL);
    return err == hipSuccess ? MHFFN_OK : MHFFN_ERR_LAUNCH;
}

int mhffn_bwd_phases(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
                     void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_dtype,
                     void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, void* stream,
                     int phases)
{
    return mhffn_bwd_layout(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_dtype, workspace, workspace_bytes, dims, dtype,
                            MHFFN_TOKENS_BHSD, stream, phases);
}

int mhffn_bwd(const void* Q, const void* K, const void* U, const void* V, const float* R, const void* dO,
              void* dQ, void* dK, void* dU, void* dV, float* dR, int grad_w_dtype,
              void* workspace, size_t workspace_bytes, const mhffn_dims* dims, int dtype, void* stream)
{
    return mhffn_bwd_phases(Q, K, U, V, R, dO, dQ, dK, dU, dV, dR, grad_w_dtype, workspace, workspace_bytes, dims,
                            dtype, stream, MHFFN_BWD_ALL);
}

static int check_gate_dims(const mhffn_dims* d)
{
    if (!d) return MHFFN_ERR_NULL_POINTER;
    if (d->B <= 0 || d->H <= 0 || d->S <= 0 || d->E <= 0 || d->d_h <= 0) return MHFFN_ERR_SHAPE;
    if (d->d_h != 64 && d->d_h != 96 && d->d_h != 128) return MHFFN_ERR_HEAD_DIM;
    if (d->E > 64 || d->B > 65535 || d->H > 65535 || (long long)d->S > (1ll << 30)) return MHFFN_ERR_SHAPE;
    if ((long long)d->B * d->H * d->S >= (1ll << 31)) return MHFFN_ERR_SHAPE;
    return MHFFN_OK;
}

int mhffn_gate_fwd(const void* X, const float* norm_weight, float eps, const float* router, void* Qn, float* R,
                   const mhffn_dims* dims, void* stream)
{
    const int rc = check_gate_dims(dims);
    if (rc != MHFFN_OK) return rc;
    if (!X || !router || !R || (norm_weight && !Qn)) return MHFFN_ERR_NULL_POINTER;
    if (!aligned16(X) || !aligned16(Qn) || !aligned16(R) || !aligned16(router) || !aligned16(norm_weight))
        return MHFFN_ERR_ALIGNMENT;
    return mhffn::launch_gate_fwd(X, norm_weight, eps, router, Qn, R, to_dims(dims), (hipStream_t)stream) == hipSuccess
               ? MHFFN_OK
               : MHFFN_ERR_LAUNCH;
}

int mhffn_gate_bwd(const void* X, const float* norm_weight, float eps, const float* router, const void* dQ,
                   int dq_token_layout, const float* dR, void* dX, float* d_norm_weight, float* d_router,
                   const mhffn_dims* dims, void* stream)
{
    const int rc = check_gate_dims(dims);
    if (rc != MHFFN_OK) return rc;
    if (dq_token_layout != MHFFN_TOKENS_BHSD && dq_token_layout != MHFFN_TOKENS_BSHD) return MHFFN_ERR_SHAPE;
    if (!X || !router || !dQ || !dR || !dX || !d_router || (norm_weight && !d_norm_weight)) return MHFFN_ERR_NULL_POINTER;
    const void* ptrs[] = {X, norm_weight, router, dQ, dR, dX, d_norm_weight, d_router};
    for (const void* p : ptrs)
        if (!aligned16(p)) return MHFFN_ERR_ALIGNMENT;
    return mhffn::launch_gate_bwd(X, norm_weight, eps, router, dQ, dq_token_layout, dR, dX, d_norm_weight, d_router,
                                  to_dims(dims), (hipStream_t)stream) == hipSuccess
               ? MHFFN_OK
               : MHFFN_ERR_LAUNCH;
}

}  // extern "C"
