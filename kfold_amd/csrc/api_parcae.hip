// C ABI: Parcae recurrence step of the trunk.
#include "../../include/kfold_hip.h"

#include "api_util.hpp"
#include "kernels.hpp"

using namespace kfh;

extern "C" {

size_t kfh_parcae_packed_bytes(int C) { return (C == 128 || C == 256) ? align_up(parcae_blob_bytes(C)) : 0; }

int kfh_parcae_pack(const void* ln_w, const void* ln_b, const void* log_a, const void* log_delta,
                    const void* b_cont, int w_dtype, int C, void* blob, void* stream_) {
    if (C != 128 && C != 256) return fail(KFH_EUNSUPPORTED, "parcae_pack: C=%d, built for C=128 and C=256", C);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "parcae_pack: bad w_dtype %d", w_dtype);
    if (!log_a || !log_delta || !b_cont || !blob) return fail(KFH_EINVAL, "parcae_pack: null pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    const size_t w_bytes = (size_t)C * C * 2;
    float* ln = reinterpret_cast<float*>(b + w_bytes);
    float* a = ln + 2 * C;
    float* b_f32 = a + C;                                    // pack-time scratch inside the blob
    launch_parcae_dynamics(log_a, log_delta, b_cont, w_dtype, a, b_f32, C, stream);
    launch_pack_blocks(b_f32, KFH_F32, C, C, C, 0, C / 32, ROW_INTERLEAVE4, K_NATURAL, 1.f, b, stream);
    launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    return check_launch("parcae_pack");
}

int kfh_parcae_step(const void* z, const void* u, const void* u_add, const void* blob, void* out,
                    long long rows, int C, float eps, int io_dtype, void* stream) {
    if (C != 128 && C != 256) return fail(KFH_EUNSUPPORTED, "parcae_step: C=%d, built for C=128 and C=256", C);
    if (rows < 0) return fail(KFH_EINVAL, "parcae_step: rows=%lld", rows);
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "parcae_step: bad io_dtype %d", io_dtype);
    if (!z || !u || !blob || !out) return fail(KFH_EINVAL, "parcae_step: null pointer argument");
    if (out == u || (u_add && out == u_add)) return fail(KFH_EINVAL, "parcae_step: out may alias z, not u");
    if (rows == 0) return KFH_OK;
    if (launch_parcae_step(z, u, u_add, io_dtype, static_cast<const char*>(blob), out, rows, C, eps,
                           static_cast<hipStream_t>(stream)) != 0)
        return fail(KFH_EUNSUPPORTED, "parcae_step: shape not built (rows=%lld C=%d)", rows, C);
    return check_launch("parcae_step");
}

}  // extern "C"
