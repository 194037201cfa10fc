// C ABI of libkfold_hip.so (declared in include/kfold_hip.h): argument checking, workspace
// carving and kernel sequencing.  No torch types, no allocation, no synchronisation.
#include "../../include/kfold_hip.h"

#include <cstdarg>
#include <cmath>
#include <cstdio>

#include "api_util.hpp"
#include "kernels.hpp"


using namespace kfh;

extern "C" {

int kfh_version(void) { return 1; }
const char* kfh_last_error(void) { return kfh::g_err; }

// ------------------------------------------------------------------------------------------
// triangle multiplication
// ------------------------------------------------------------------------------------------
namespace {
bool trimul_wide(int C) { return C == 256; }
// any other multiple of 32 up to 256 runs on the path assembled from the token-track kernels
bool trimul_generic(int C) { return C != kC && !trimul_wide(C) && trimul_generic_blob_bytes(C) != 0; }
}  // namespace

size_t kfh_trimul_packed_bytes(int C) {
    if (trimul_wide(C)) return align_up(trimul_wide_blob_bytes(C));
    if (trimul_generic(C)) return trimul_generic_blob_bytes(C);
    return C == kC ? align_up(kTmBlobBytes) : 0;
}

int kfh_trimul_pack(const void* ln_in_w, const void* ln_in_b, const void* p_in_w,
                    const void* g_in_w, const void* ln_out_w, const void* ln_out_b,
                    const void* p_out_w, const void* g_out_w, int w_dtype, int C, void* blob,
                    void* stream_) {
    if (C != kC && !trimul_wide(C) && !trimul_generic(C))
        return fail(KFH_EUNSUPPORTED, "trimul_pack: C=%d (a multiple of 32 up to 256)", C);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "trimul_pack: bad w_dtype %d", w_dtype);
    if (!p_in_w || !g_in_w || !p_out_w || !g_out_w || !blob)
        return fail(KFH_EINVAL, "trimul_pack: null weight or blob pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    if (trimul_generic(C)) {
        if (trimul_generic_pack(ln_in_w, ln_in_b, p_in_w, g_in_w, ln_out_w, ln_out_b, p_out_w, g_out_w, w_dtype, C,
                                blob, stream))
            return fail(KFH_EUNSUPPORTED, "trimul_pack: C=%d not built", C);
        return check_launch("trimul_pack");
    }
    if (trimul_wide(C)) {
        size_t o_gate, o_ab, o_out, o_ln, blk;
        trimul_wide_offsets(C, &o_gate, &o_ab, &o_out, &o_ln, &blk);
        for (int cb = 0; cb < 2 * C / 32; ++cb) {
            launch_pack_blocks(p_in_w, w_dtype, 32, C, C, 32 * cb, 1, ROW_NATURAL, K_NATURAL, 1.f,
                               b + o_ab + (2 * cb) * blk, stream);
            launch_pack_blocks(g_in_w, w_dtype, 32, C, C, 32 * cb, 1, ROW_NATURAL, K_NATURAL, -kLog2e,
                               b + o_ab + (2 * cb + 1) * blk, stream);
        }
        launch_pack_blocks(g_out_w, w_dtype, C, C, C, 0, C / 32, ROW_INTERLEAVE4, K_NATURAL, -kLog2e, b + o_gate,
                           stream);
        launch_pack_blocks(p_out_w, w_dtype, C, C, C, 0, C / 32, ROW_INTERLEAVE4, K_HALF, 1.f, b + o_out, stream);
        float* lnw = reinterpret_cast<float*>(b + o_ln);
        launch_copy_f32(ln_in_w, w_dtype, lnw, C, 1.f, stream);
        launch_copy_f32(ln_in_b, w_dtype, lnw + C, C, 0.f, stream);
        launch_copy_f32(ln_out_w, w_dtype, lnw + 2 * C, C, 1.f, stream);
        launch_copy_f32(ln_out_b, w_dtype, lnw + 3 * C, C, 0.f, stream);
        return check_launch("trimul_pack");
    }
    // input phase: step cb = { p_in rows 32cb.., g_in rows 32cb.. }
    for (int cb = 0; cb < 8; ++cb) {
        launch_pack_blocks(p_in_w, w_dtype, 32, C, C, 32 * cb, 1, ROW_NATURAL, K_NATURAL, 1.f,
                           b + kTmAbOff + (2 * cb) * kBlockBytes, stream);
        launch_pack_blocks(g_in_w, w_dtype, 32, C, C, 32 * cb, 1, ROW_NATURAL, K_NATURAL, -kLog2e,
                           b + kTmAbOff + (2 * cb + 1) * kBlockBytes, stream);
    }
    launch_pack_blocks(g_out_w, w_dtype, C, C, C, 0, 4, ROW_INTERLEAVE4, K_NATURAL, -kLog2e,
                       b + kTmGateOff, stream);
    launch_pack_blocks(p_out_w, w_dtype, C, C, C, 0, 4, ROW_INTERLEAVE4, K_HALF, 1.f, b + kTmOutOff,
                       stream);
    float* ln = reinterpret_cast<float*>(b + kTmLnOff);
    launch_copy_f32(ln_in_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_in_b, w_dtype, ln + C, C, 0.f, stream);
    launch_copy_f32(ln_out_w, w_dtype, ln + 2 * C, C, 1.f, stream);
    launch_copy_f32(ln_out_b, w_dtype, ln + 3 * C, C, 0.f, stream);
    return check_launch("trimul_pack");
}

size_t kfh_trimul_workspace_bytes(int N, int C) {
    if (trimul_generic(C)) return trimul_generic_ws_bytes(N, C);
    if ((C != kC && !trimul_wide(C)) || N <= 0) return 0;
    const size_t np = trimul_np(N);
    const size_t planes_ab = align_up(2 * (size_t)C * np * np * 2);
    const size_t planes_y = align_up((size_t)C * np * np * 2);
    return planes_ab + planes_y;
}

size_t kfh_trimul_workspace_bytes_batched(int B, int N, int C) {
    if (B <= 0) return 0;
    if (trimul_generic(C)) return trimul_generic_ws_bytes(N, C, B);
    return kfh_trimul_workspace_bytes(N, C);
}

int kfh_trimul_forward(const void* z, const uint8_t* mask, const void* blob, const void* residual,
                       void* out, void* workspace, size_t workspace_bytes, int B, int N, int C,
                       int direction, float eps, int io_dtype, void* stream) {
    return kfh_trimul_forward_stages(z, mask, blob, residual, out, workspace, workspace_bytes, B, N, C,
                                     direction, eps, io_dtype, KFH_STAGE_ALL, stream);
}

int kfh_trimul_forward_stages(const void* z, const uint8_t* mask, const void* blob,
                              const void* residual, void* out, void* workspace,
                              size_t workspace_bytes, int B, int N, int C, int direction, float eps,
                              int io_dtype, int stages, void* stream_) {
    return kfh_trimul_forward_rows(z, mask, blob, residual, out, workspace, workspace_bytes, B, N, C, direction,
                                   eps, io_dtype, stages, 0, N, stream_);
}

int kfh_trimul_row_granule(int N, int C) {
    if ((C != kC && !trimul_wide(C)) || N <= 0) return 0;
    return contract_tile_rows(trimul_np(N));
}

int kfh_trimul_forward_rows(const void* z, const uint8_t* mask, const void* blob,
                            const void* residual, void* out, void* workspace,
                            size_t workspace_bytes, int B, int N, int C, int direction, float eps,
                            int io_dtype, int stages, int row0, int nrows, void* stream_) {
    if (C != kC && !trimul_wide(C) && !trimul_generic(C))
        return fail(KFH_EUNSUPPORTED, "trimul_forward: C=%d (a multiple of 32 up to 256)", C);
    if (B <= 0 || N <= 0) return fail(KFH_EINVAL, "trimul_forward: bad shape B=%d N=%d", B, N);
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "trimul_forward: bad io_dtype %d", io_dtype);
    if (direction != KFH_OUTGOING && direction != KFH_INCOMING)
        return fail(KFH_EINVAL, "trimul_forward: bad direction %d", direction);
    if (!z || !mask || !blob || !out || !workspace)
        return fail(KFH_EINVAL, "trimul_forward: null pointer argument");
    if (out == z && residual != z)
        return fail(KFH_EINVAL, "trimul_forward: out may alias z only when residual == z");
    const bool ranged = row0 != 0 || nrows != N;
    if (ranged) {
        const int granule = kfh_trimul_row_granule(N, C);
        if (granule == 0 || B != 1)
            return fail(KFH_EUNSUPPORTED, "trimul_forward_rows: row ranges take B = 1 and C = 128 or 256 (B=%d C=%d)", B, C);
        if (row0 < 0 || nrows < 0 || row0 + nrows > N || row0 % granule || (nrows % granule && row0 + nrows != N))
            return fail(KFH_EINVAL, "trimul_forward_rows: rows [%d, %d) of %d (ranges start at multiples of %d)", row0,
                        row0 + nrows, N, granule);
    }
    const size_t need = kfh_trimul_workspace_bytes(N, C);
    if (workspace_bytes < need)
        return fail(KFH_EINVAL, "trimul_forward: workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int np = trimul_np(N);
    const size_t esz = io_dtype == KFH_F32 ? 4 : 2;
    char* ws = static_cast<char*>(workspace);
    if (trimul_generic(C)) {
        // a workspace of kfh_trimul_workspace_bytes_batched(B, N, C) takes all batch elements
        // (templates) through every kernel at once; a smaller one takes them in turn
        const bool folded = B > 1 && workspace_bytes >= trimul_generic_ws_bytes(N, C, B);
        const int step = folded ? B : 1;
        for (int b = 0; b < B; b += step) {
            const size_t off = (size_t)b * N * N * C * esz;
            const int rc = trimul_generic_forward(
                static_cast<const char*>(z) + off, io_dtype, mask + (size_t)b * N * N, static_cast<const char*>(blob),
                ws, residual ? static_cast<const char*>(residual) + off : nullptr, static_cast<char*>(out) + off, step,
                N, C, direction == KFH_INCOMING, eps, stages, stream);
            if (rc) return fail(KFH_EUNSUPPORTED, "trimul_forward: shape not built (%d)", rc);
        }
        return check_launch("trimul_forward");
    }
    uint16_t* planes_ab = reinterpret_cast<uint16_t*>(ws);
    uint16_t* planes_y = reinterpret_cast<uint16_t*>(ws + align_up(2 * (size_t)C * np * np * 2));
    const char* bl = static_cast<const char*>(blob);
    for (int b = 0; b < B; ++b) {
        const size_t off = (size_t)b * N * N * C * esz;
        const char* zb = static_cast<const char*>(z) + off;
        const char* rb = residual ? static_cast<const char*>(residual) + off : nullptr;
        char* ob = static_cast<char*>(out) + off;
        if (stages & KFH_STAGE_IN) {
            if (trimul_wide(C))
                launch_trimul_in_wide(zb, io_dtype, mask + (size_t)b * N * N, bl, planes_ab, N, np, C,
                                      direction == KFH_INCOMING, eps, stream);
            else
                launch_trimul_in(zb, io_dtype, mask + (size_t)b * N * N, bl, planes_ab, N, np,
                                 direction == KFH_INCOMING, eps, stream);
        }
        // the input phase always makes all rows of the planes; the last range of the contraction
        // also takes the padded rows below N
        const int crows = row0 + nrows == N ? np - row0 : nrows;
        if (stages & KFH_STAGE_CORE)
            launch_contract(planes_ab, planes_ab + (size_t)C * np * np, planes_y, np, C, stream, row0, crows);
        if (stages & KFH_STAGE_OUT) {
            if (trimul_wide(C))
                launch_trimul_out_wide(planes_y, zb, bl, rb, ob, io_dtype, N, np, C, eps, stream, row0, nrows);
            else
                launch_trimul_out(planes_y, zb, bl, rb, ob, io_dtype, N, np, eps, stream, row0, nrows);
        }
    }
    return check_launch("trimul_forward");
}

// ------------------------------------------------------------------------------------------
// triangle attention
// ------------------------------------------------------------------------------------------
namespace {
struct TaSizes { size_t frag, bias, codes, total; int nb; };
TaSizes ta_sizes(int N) {
    TaSizes s;
    s.nb = (N + 31) / 32;
    s.frag = align_up((size_t)N * 4 * s.nb * 2048);
    s.bias = align_up((size_t)4 * s.nb * s.nb * 2048);
    s.codes = align_up((size_t)N * s.nb * 32);
    s.total = 4 * s.frag + s.bias + s.codes;
    return s;
}
}  // namespace

namespace {
bool triattn_fused(int C, int H) { return C == kC && H == 4; }
}  // namespace

size_t kfh_triattn_packed_bytes(int C, int H) {
    return triattn_fused(C, H) ? align_up(kTaBlobBytes) : triattn_generic_blob_bytes(C, H);
}

int kfh_triattn_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* k_w,
                     const void* v_w, const void* g_w, const void* bias_w, const void* o_w,
                     int w_dtype, int C, int H, void* blob, void* stream_) {
    if (!triattn_fused(C, H) && triattn_generic_blob_bytes(C, H) == 0)
        return fail(KFH_EUNSUPPORTED, "triattn_pack: C=%d H=%d (C a multiple of 32, head dim <= 64)", C, H);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "triattn_pack: bad w_dtype %d", w_dtype);
    if (!q_w || !k_w || !v_w || !g_w || !bias_w || !o_w || !blob)
        return fail(KFH_EINVAL, "triattn_pack: null weight or blob pointer");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!triattn_fused(C, H)) {
        if (triattn_generic_pack(ln_w, ln_b, q_w, k_w, v_w, g_w, bias_w, o_w, w_dtype, C, H, blob, stream))
            return fail(KFH_EUNSUPPORTED, "triattn_pack: C=%d H=%d not built", C, H);
        return check_launch("triattn_pack");
    }
    char* b = static_cast<char*>(blob);
    const float qscale = kLog2e / sqrtf((float)(C / H));
    for (int h = 0; h < 4; ++h) {
        launch_pack_blocks(q_w, w_dtype, 32, C, C, 32 * h, 1, ROW_NATURAL, K_NATURAL, qscale,
                           b + kTaProjOff + (2 * h) * kBlockBytes, stream);
        launch_pack_blocks(k_w, w_dtype, 32, C, C, 32 * h, 1, ROW_NATURAL, K_NATURAL, 1.f,
                           b + kTaProjOff + (2 * h + 1) * kBlockBytes, stream);
        launch_pack_blocks(v_w, w_dtype, 32, C, C, 32 * h, 1, ROW_NATURAL, K_NATURAL, 1.f,
                           b + kTaProjOff + (8 + h) * kBlockBytes, stream);
        launch_pack_blocks(g_w, w_dtype, 32, C, C, 32 * h, 1, ROW_NATURAL, K_NATURAL, -kLog2e,
                           b + kTaGateOff + h * kBlockBytes, stream);
    }
    launch_pack_blocks(bias_w, w_dtype, H, C, C, 0, 1, ROW_NATURAL, K_NATURAL, kLog2e,
                       b + kTaProjOff + 12 * kBlockBytes, stream);
    launch_fill_zero(b + kTaProjOff + 13 * kBlockBytes, kBlockBytes, stream);
    launch_pack_blocks(o_w, w_dtype, C, C, C, 0, 4, ROW_INTERLEAVE4, K_ACC, 1.f, b + kTaOutOff, stream);
    float* ln = reinterpret_cast<float*>(b + kTaLnOff);
    launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    return check_launch("triattn_pack");
}

size_t kfh_triattn_workspace_bytes(int N, int C, int H) {
    if (N <= 0 || N > 8192) return 0;
    if (!triattn_fused(C, H)) return triattn_generic_ws_bytes(N, C, H);
    return ta_sizes(N).total;
}

size_t kfh_triattn_workspace_bytes_batched(int B, int N, int C, int H) {
    if (B <= 0 || N <= 0 || N > 8192) return 0;
    if (!triattn_fused(C, H)) return triattn_generic_ws_bytes(N, C, H, B);
    return ta_sizes(N).total;
}

int kfh_triattn_forward(const void* x, const uint8_t* mask, const void* blob, const void* residual,
                        void* out, void* workspace, size_t workspace_bytes, int B, int N, int C,
                        int H, int ending, float eps, int io_dtype, void* stream) {
    return kfh_triattn_forward_stages(x, mask, blob, residual, out, workspace, workspace_bytes, B, N, C,
                                      H, ending, eps, io_dtype, KFH_STAGE_ALL, stream);
}

int kfh_triattn_forward_stages(const void* x, const uint8_t* mask, const void* blob,
                               const void* residual, void* out, void* workspace,
                               size_t workspace_bytes, int B, int N, int C, int H, int ending,
                               float eps, int io_dtype, int stages, void* stream_) {
    return kfh_triattn_forward_rows(x, mask, blob, residual, out, workspace, workspace_bytes, B, N, C, H, ending,
                                    eps, io_dtype, stages, 0, N, stream_);
}

int kfh_triattn_forward_rows(const void* x, const uint8_t* mask, const void* blob,
                             const void* residual, void* out, void* workspace,
                             size_t workspace_bytes, int B, int N, int C, int H, int ending,
                             float eps, int io_dtype, int stages, int row0, int nrows, void* stream_) {
    if (!triattn_fused(C, H) && triattn_generic_blob_bytes(C, H) == 0)
        return fail(KFH_EUNSUPPORTED, "triattn_forward: C=%d H=%d (C a multiple of 32, head dim <= 64)", C, H);
    if (B <= 0 || N <= 0) return fail(KFH_EINVAL, "triattn_forward: bad shape B=%d N=%d", B, N);
    if (N > 8192) return fail(KFH_EUNSUPPORTED, "triattn_forward: N=%d > 8192", N);
    if (!dtype_ok(io_dtype)) return fail(KFH_EINVAL, "triattn_forward: bad io_dtype %d", io_dtype);
    if (!x || !mask || !blob || !out || !workspace)
        return fail(KFH_EINVAL, "triattn_forward: null pointer argument");
    if (out == x && residual != x)
        return fail(KFH_EINVAL, "triattn_forward: out may alias x only when residual == x");
    if (row0 != 0 || nrows != N) {
        if (!triattn_fused(C, H) || B != 1)
            return fail(KFH_EUNSUPPORTED, "triattn_forward_rows: row ranges take B = 1, C = 128, H = 4 (B=%d C=%d H=%d)", B, C, H);
        if (row0 < 0 || nrows < 0 || row0 + nrows > N)
            return fail(KFH_EINVAL, "triattn_forward_rows: rows [%d, %d) of %d", row0, row0 + nrows, N);
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!triattn_fused(C, H)) {
        const size_t need = triattn_generic_ws_bytes(N, C, H);
        if (workspace_bytes < need)
            return fail(KFH_EINVAL, "triattn_forward: workspace %zu < %zu bytes", workspace_bytes, need);
        const size_t esz_g = io_dtype == KFH_F32 ? 4 : 2;
        // a workspace of kfh_triattn_workspace_bytes_batched(B, N, C, H) takes all batch elements
        // (templates) through the projection kernels at once; a smaller one takes them in turn
        const bool folded = B > 1 && workspace_bytes >= triattn_generic_ws_bytes(N, C, H, B);
        const int step = folded ? B : 1;
        for (int b = 0; b < B; b += step) {
            const size_t off = (size_t)b * N * N * C * esz_g;
            const int rc = triattn_generic_forward(
                static_cast<const char*>(x) + off, io_dtype, mask + (size_t)b * N * N, static_cast<const char*>(blob),
                static_cast<char*>(workspace), residual ? static_cast<const char*>(residual) + off : nullptr,
                static_cast<char*>(out) + off, step, N, C, H, ending, eps, stages, stream);
            if (rc) return fail(KFH_EUNSUPPORTED, "triattn_forward: shape not built (%d)", rc);
        }
        return check_launch("triattn_forward");
    }
    const TaSizes sz = ta_sizes(N);
    if (workspace_bytes < sz.total)
        return fail(KFH_EINVAL, "triattn_forward: workspace %zu < %zu bytes", workspace_bytes, sz.total);
    char* w = static_cast<char*>(workspace);
    TriattnWorkspace ws;
    ws.qf = w; ws.kf = w + sz.frag; ws.vf = w + 2 * sz.frag; ws.of = w + 3 * sz.frag;
    ws.biast = reinterpret_cast<uint16_t*>(w + 4 * sz.frag);
    ws.codes = reinterpret_cast<uint8_t*>(w + 4 * sz.frag + sz.bias);
    const size_t esz = io_dtype == KFH_F32 ? 4 : 2;
    for (int b = 0; b < B; ++b) {
        const size_t off = (size_t)b * N * N * C * esz;
        if ((stages & KFH_STAGE_IN) && N % 32) {
            // queries beyond N in the last query block have no projected bias: keep their tiles finite
            for (int h = 0; h < 4; ++h)
                launch_fill_zero(ws.biast + (((size_t)h * sz.nb + (sz.nb - 1)) * sz.nb) * kBiasTileElems,
                                 (size_t)sz.nb * 2048, stream);
        }
        const int rc = launch_triattn(static_cast<const char*>(x) + off, io_dtype, mask + (size_t)b * N * N,
                                      static_cast<const char*>(blob), ws,
                                      residual ? static_cast<const char*>(residual) + off : nullptr,
                                      static_cast<char*>(out) + off, N, ending, eps, stages, stream, row0, nrows);
        if (rc == -3)
            return fail(KFH_EINVAL, "triattn_forward_rows: a range of %d rows is too short for the attention kernel of "
                        "N = %d (48 rows at least)", nrows, N);
        if (rc) return fail(KFH_EHIP, "triattn_forward: attention kernel launch failed (%d)", rc);
    }
    return check_launch("triattn_forward");
}

size_t kfh_pair_block_workspace_bytes(int B, int N, int C, int H, int expansion) {
    if (B <= 0) return 0;
    // the sizes that take a batch through the kernels at once where the path can
    const size_t a = kfh_trimul_workspace_bytes_batched(B, N, C), b = kfh_triattn_workspace_bytes_batched(B, N, C, H);
    if (a == 0 || b == 0 || kfh_transition_packed_bytes(C, expansion) == 0) return 0;
    const size_t c = kfh_transition_workspace_bytes((long long)B * N * N, C, expansion);
    return a > b ? (a > c ? a : c) : (b > c ? b : c);
}

int kfh_pair_block_forward(void* z, const uint8_t* pair_mask, const void* trimul_out_blob,
                           const void* trimul_in_blob, const void* triattn_start_blob,
                           const void* triattn_end_blob, const void* transition_blob, void* workspace,
                           size_t workspace_bytes, int B, int N, int C, int H, int expansion, float eps,
                           int io_dtype, void* stream) {
    const size_t need = kfh_pair_block_workspace_bytes(B > 0 ? B : 1, N, C, H, expansion);
    if (need == 0)
        return fail(KFH_EUNSUPPORTED, "pair_block_forward: C=%d H=%d expansion=%d N=%d not supported", C, H, expansion, N);
    if (B <= 0) return fail(KFH_EINVAL, "pair_block_forward: bad shape B=%d N=%d", B, N);
    if (!z || !pair_mask || !trimul_out_blob || !trimul_in_blob || !triattn_start_blob || !triattn_end_blob ||
        !transition_blob || !workspace)
        return fail(KFH_EINVAL, "pair_block_forward: null pointer argument");
    if (workspace_bytes < need)
        return fail(KFH_EINVAL, "pair_block_forward: workspace %zu < %zu bytes", workspace_bytes, need);
    // the five in-place updates of the reference's eval-mode block, each with its residual fused
    int rc = kfh_trimul_forward(z, pair_mask, trimul_out_blob, z, z, workspace, workspace_bytes, B, N, C,
                                KFH_OUTGOING, eps, io_dtype, stream);
    if (rc) return rc;
    rc = kfh_trimul_forward(z, pair_mask, trimul_in_blob, z, z, workspace, workspace_bytes, B, N, C, KFH_INCOMING,
                            eps, io_dtype, stream);
    if (rc) return rc;
    rc = kfh_triattn_forward(z, pair_mask, triattn_start_blob, z, z, workspace, workspace_bytes, B, N, C, H, 0, eps,
                             io_dtype, stream);
    if (rc) return rc;
    rc = kfh_triattn_forward(z, pair_mask, triattn_end_blob, z, z, workspace, workspace_bytes, B, N, C, H, 1, eps,
                             io_dtype, stream);
    if (rc) return rc;
    return kfh_transition_forward(z, transition_blob, z, pair_mask, z, workspace, workspace_bytes,
                                  (long long)B * N * N, C, expansion, eps, io_dtype, stream);
}

}  // extern "C"
