// Triangle multiplication for pair widths other than the fused C = 128 / 256 paths (the
// reference's apo template stack runs its whole Pairformer block at C = 64:
// configs/kfold.yaml:15-19, model/modules/apo_module.py:107-172, :294-301).  Same math
// (model/primitives/triangle_multiplication.py:212-229, :296-313), assembled from the token-track
// building blocks and the contraction kernel:
//     rows_norm            xn = LN_in(z)                        [N^2, C] bf16
//     linear EPI_PLANES    ab = (Wp xn) * sigmoid(Wg xn) * mask -> channel-major planes ab[2C][Np][Np]
//     contract_kernel      y_d = a_d b_d^T                      (contract.hip)
//     planes_norm          yn = LN_out(y)                       [N^2, C] bf16
//     linear EPI_SIGMOID   gate = sigmoid(Wg_out xn)
//     linear EPI_RESID     out = (residual +) gate * (Wp_out yn)
// The incoming direction runs the same sequence in transposed row order (xn is written
// transposed, so plane[d][i][k] = ab[k, i, d] is again a contiguous store and the contraction the
// same NT product) and transposes the output rows back in the last kernel.
#include "api_util.hpp"
#include "kernels.hpp"

namespace kfh {

namespace {
struct TmgLayout {
    int C;
    size_t w_pin, w_gin, w_gout, w_pout, ln, total;
    bool ok;
    explicit TmgLayout(int C_) : C(C_) {
        ok = C > 0 && C % 32 == 0 && C <= 256;
        total = 0;
        if (!ok) return;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        const size_t blk = (size_t)(C / 16) * 1024;          // one packed 32-row block of C channels
        w_pin = take((size_t)(2 * C / 32) * blk);
        w_gin = take((size_t)(2 * C / 32) * blk);
        w_gout = take((size_t)(C / 32) * blk);
        w_pout = take((size_t)(C / 32) * blk);
        ln = take(4 * (size_t)C * 4);
        total = off;
    }
};
struct TmgWs {
    size_t xn, ab, y, yn, gate, total;
    int np;
    TmgWs(const TmgLayout& l, int N, int B) {
        np = trimul_np(N);
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        xn = take((size_t)B * N * N * l.C * 2);
        ab = take((size_t)B * 2 * l.C * np * np * 2);      // [a planes of all elements][b planes of all elements]
        y = take((size_t)B * l.C * np * np * 2);
        yn = take((size_t)B * N * N * l.C * 2);
        gate = take((size_t)B * N * N * l.C * 2);
        total = off;
    }
};

// yn[b][row(i, j)][c] = LN_out over c of y[b * C + c][i][j] (fp32 statistics, biased variance), bf16;
// one thread per position, three passes over its C plane values (the second and third hit L2).
// transposed: row(i, j) = j * N + i, else i * N + j.
__global__ __launch_bounds__(256) void planes_norm_kernel(const uint16_t* __restrict__ planes,
                                                          const float* __restrict__ gamma,
                                                          const float* __restrict__ beta,
                                                          uint16_t* __restrict__ out, int B, int N, int Np, int C,
                                                          float eps, int transposed) {
    long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)B * N * N) return;
    const int b = (int)(idx / ((long long)N * N));
    idx -= (long long)b * N * N;
    const int i = (int)(idx / N), j = (int)(idx % N);
    const size_t plane_sz = (size_t)Np * Np, pi = (size_t)i * Np + j;
    planes += (size_t)b * C * plane_sz;
    out += (size_t)b * N * N * C;
    float s = 0.f;
    for (int c = 0; c < C; ++c) s += bf16_lo(planes[c * plane_sz + pi]);
    const float mean = s / C;
    float q = 0.f;
    for (int c = 0; c < C; ++c) {
        const float d = bf16_lo(planes[c * plane_sz + pi]) - mean;
        q += d * d;
    }
    const float rstd = __builtin_amdgcn_rsqf(q / C + eps);
    uint16_t* dst = out + (size_t)(transposed ? (size_t)j * N + i : (size_t)i * N + j) * C;
    for (int c = 0; c < C; c += 2) {
        const float a = (bf16_lo(planes[c * plane_sz + pi]) - mean) * rstd * gamma[c] + beta[c];
        const float b = (bf16_lo(planes[(c + 1) * plane_sz + pi]) - mean) * rstd * gamma[c + 1] + beta[c + 1];
        *reinterpret_cast<uint32_t*>(dst + c) = pack_bf16(a, b);
    }
}
}  // namespace

size_t trimul_generic_blob_bytes(int C) { return TmgLayout(C).total; }
size_t trimul_generic_ws_bytes(int N, int C, int B) {
    const TmgLayout l(C);
    if (!l.ok || N <= 0 || B <= 0) return 0;
    return TmgWs(l, N, B).total;
}

int trimul_generic_pack(const void* ln_in_w, const void* ln_in_b, const void* p_in_w, const void* g_in_w,
                        const void* ln_out_w, const void* ln_out_b, const void* p_out_w, const void* g_out_w,
                        int w_dtype, int C, void* blob, hipStream_t stream) {
    const TmgLayout l(C);
    if (!l.ok) return -1;
    char* b = static_cast<char*>(blob);
    launch_pack_blocks(p_in_w, w_dtype, 2 * C, C, C, 0, 2 * C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_pin, stream);
    launch_pack_blocks(g_in_w, w_dtype, 2 * C, C, C, 0, 2 * C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_gin, stream);
    launch_pack_blocks(g_out_w, w_dtype, C, C, C, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_gout, stream);
    launch_pack_blocks(p_out_w, w_dtype, C, C, C, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f, b + l.w_pout, stream);
    float* ln = reinterpret_cast<float*>(b + l.ln);
    launch_copy_f32(ln_in_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_in_b, w_dtype, ln + C, C, 0.f, stream);
    launch_copy_f32(ln_out_w, w_dtype, ln + 2 * C, C, 1.f, stream);
    launch_copy_f32(ln_out_b, w_dtype, ln + 3 * C, C, 0.f, stream);
    return 0;
}

// B batch elements folded into the rows of every kernel (row group a = b * N + i); returns 0 or a
// negative code of the failing launch helper
int trimul_generic_forward(const void* z, int io_dtype, const uint8_t* mask, const char* blob, char* ws,
                           const void* residual, void* out, int B, int N, int C, int incoming, float eps,
                           int stages, hipStream_t stream) {
    const TmgLayout l(C);
    if (!l.ok || B <= 0) return -1;
    if ((long long)B * N > 0x7fffffffLL / 64) return -1;
    const TmgWs w(l, N, B);
    const long long rows = (long long)B * N * N;
    const int nb = (N + 31) / 32;
    const size_t plane_sz = (size_t)w.np * w.np;
    uint16_t* xn = reinterpret_cast<uint16_t*>(ws + w.xn);
    uint16_t* ab = reinterpret_cast<uint16_t*>(ws + w.ab);
    uint16_t* y = reinterpret_cast<uint16_t*>(ws + w.y);
    uint16_t* yn = reinterpret_cast<uint16_t*>(ws + w.yn);
    const float* ln = reinterpret_cast<const float*>(blob + l.ln);
    auto base = [&](const void* A, const void* W, int nout) {
        LinearArgs p{};
        p.A = A; p.lda = C; p.rows_a = B * N; p.L = N; p.nb = nb; p.K = C; p.W = W; p.nblk = nout / 32; p.Nout = nout;
        p.bias_scale = 1.f; p.H = 1; p.PB = 1; p.Dh = 32;
        p.batch_rows = N; p.nbatch = B; p.plane_side = C;
        return p;
    };
    if (stages & KFH_STAGE_IN) {
        // rows (a, pos): outgoing (i, k) = z[i, k]; incoming (i, k) = z[k, i] (written transposed)
        if (launch_rows_norm(z, io_dtype, ln, ln + C, xn, rows, C, 1, eps, stream, incoming ? N : 0)) return -2;
        if (w.np != N) launch_fill_zero(ab, (size_t)B * 2 * C * plane_sz * 2, stream);      // zero padding of the planes
        LinearArgs p = base(xn, blob + l.w_pin, 2 * C);
        p.W2 = blob + l.w_gin;
        p.epi = EPI_PLANES; p.out = ab; p.ldo = w.np;
        p.mask = mask; p.mask_transposed = incoming ? 1 : 0;
        if (launch_linear(p, stream)) return -3;
    }
    if (stages & KFH_STAGE_CORE)      // one NT product per (element, channel): B * C planes on each side
        launch_contract(ab, ab + (size_t)B * C * plane_sz, y, w.np, B * C, stream);
    if (stages & KFH_STAGE_OUT) {
        // transposed row order for the incoming direction: row (j, i) holds position (i, j)
        hipLaunchKernelGGL(planes_norm_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream, y,
                           ln + 2 * C, ln + 3 * C, yn, B, N, w.np, C, eps, incoming ? 1 : 0);
        LinearArgs g = base(xn, blob + l.w_gout, C);
        g.epi = EPI_SIGMOID; g.out = ws + w.gate; g.out_dtype = KFH_BF16; g.ldo = C;
        if (launch_linear(g, stream)) return -3;
        LinearArgs p = base(yn, blob + l.w_pout, C);
        p.epi = EPI_RESID;
        p.gate = reinterpret_cast<const uint16_t*>(ws + w.gate); p.ld_gate = C;
        p.out_transposed = incoming ? 1 : 0;
        if (residual) { p.aux = residual; p.aux_dtype = io_dtype; p.ld_aux = C; }
        p.out = out; p.out_dtype = io_dtype; p.ldo = C;
        if (launch_linear(p, stream)) return -3;
    }
    return 0;
}

}  // namespace kfh
