// Triangle attention for pair widths / head shapes other than the fused C = 128, 4 x 32 path
// (the reference's apo stack runs C = 64, 4 heads x 16, batched over templates:
// configs/kfold.yaml:15-19, model/modules/apo_module.py:376-384).  Same math
// (model/primitives/triangle_attention.py:375-434, :246-335), assembled from the token-track
// building blocks: row LayerNorm, MFMA linears into fragment order, the shared-bias attention
// kernels of flash.hip (head dim zero-padded to 32 or 64) and an MFMA output projection.  The
// ending node is handled by writing the normalised rows transposed and transposing the output
// rows back in the last kernel; no transposed copy of x is made.
#include <cmath>

#include "api_util.hpp"
#include "kernels.hpp"

namespace kfh {

namespace {
struct TagLayout {
    int C, H, Dh, PB, kq, nhb, ko;
    size_t wq, wk, wv, wg, wo, wb, ln, total;
    bool ok;
    TagLayout(int C_, int H_) : C(C_), H(H_) {
        ok = C > 0 && H > 0 && C % H == 0 && C % 32 == 0 && C <= 2048 && H <= 32;
        total = 0;
        if (!ok) return;
        Dh = C / H;
        PB = (Dh + 31) / 32;
        ok = PB <= 2;
        if (!ok) return;
        kq = C / 16; nhb = H * PB; ko = nhb * 2;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        const size_t wh = (size_t)nhb * kq * 1024;
        wq = take(wh); wk = take(wh); wv = take(wh); wg = take(wh);
        wo = take((size_t)(C / 32) * ko * 1024);
        wb = take((size_t)kq * 1024);
        ln = take(2 * (size_t)C * 4);
        total = off;
    }
};
struct TagWs {
    size_t xn, qf, kf, vf, gf, of, bias, tiles, codes, total;
    size_t frag1, tiles1, codes1;       // bytes of one batch element's fragments / bias tiles / key codes
    int nb;
    TagWs(const TagLayout& l, int N, int B) {
        nb = (N + 31) / 32;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        xn = take((size_t)B * N * N * l.C * 2);
        frag1 = (size_t)N * l.H * nb * l.PB * 2048;
        qf = take(B * frag1); kf = take(B * frag1); vf = take(B * frag1); gf = take(B * frag1); of = take(B * frag1);
        bias = take((size_t)B * N * N * l.H * 2);
        tiles1 = (size_t)l.H * nb * nb * 2048;
        tiles = take(B * tiles1);
        codes1 = (size_t)N * nb * 32;
        codes = take(B * codes1);
        total = off;
    }
};
}  // namespace

size_t triattn_generic_blob_bytes(int C, int H) { return TagLayout(C, H).total; }
size_t triattn_generic_ws_bytes(int N, int C, int H, int B) {
    const TagLayout l(C, H);
    if (!l.ok || N <= 0 || N > 8192 || B <= 0) return 0;
    return TagWs(l, N, B).total;
}

int triattn_generic_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* k_w, const void* v_w,
                         const void* g_w, const void* bias_w, const void* o_w, int w_dtype, int C, int H,
                         void* blob, hipStream_t stream) {
    const TagLayout l(C, H);
    if (!l.ok) return -1;
    char* b = static_cast<char*>(blob);
    const float qscale = kLog2e / sqrtf((float)l.Dh);
    const size_t blk = (size_t)l.kq * 1024;
    for (int h = 0; h < H; ++h)
        for (int pp = 0; pp < l.PB; ++pp) {
            const int rows = l.Dh - 32 * pp < 32 ? l.Dh - 32 * pp : 32;
            const int row0 = h * l.Dh + 32 * pp;
            const size_t o = (size_t)(h * l.PB + pp) * blk;
            launch_pack_blocks(q_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, qscale, b + l.wq + o, stream);
            launch_pack_blocks(k_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wk + o, stream);
            launch_pack_blocks(v_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wv + o, stream);
            launch_pack_blocks(g_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wg + o, stream);
        }
    launch_pack_blocks(o_w, w_dtype, C, l.ko * 16, C, 0, C / 32, ROW_NATURAL, K_ACC_HEADPAD, 1.f, b + l.wo, stream,
                       l.Dh | ((2 * l.PB) << 16));
    launch_pack_blocks(bias_w, w_dtype, H, C, C, 0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wb, stream);
    float* ln = reinterpret_cast<float*>(b + l.ln);
    launch_copy_f32(ln_w, w_dtype, ln, C, 1.f, stream);
    launch_copy_f32(ln_b, w_dtype, ln + C, C, 0.f, stream);
    return 0;
}

// B batch elements: LayerNorm, projections, bias and the output projection run over the rows of all
// elements at once (row group a = b * N + i); the attention core is launched per element (its
// pair bias is the element's).  Returns 0 or a negative code of the failing launch helper.
int triattn_generic_forward(const void* x, int io_dtype, const uint8_t* mask, const char* blob, char* ws,
                            const void* residual, void* out, int B, int N, int C, int H, int ending, float eps,
                            int stages, hipStream_t stream) {
    const TagLayout l(C, H);
    if (!l.ok || B <= 0) return -1;
    if ((long long)B * N > 0x7fffffffLL / 64) return -1;
    const TagWs w(l, N, B);
    const long long rows = (long long)B * N * N;
    uint16_t* xn = reinterpret_cast<uint16_t*>(ws + w.xn);
    const float* ln = reinterpret_cast<const float*>(blob + l.ln);
    auto base = [&](const void* A, long long lda, int K) {
        LinearArgs p{};
        p.A = A; p.lda = lda; p.rows_a = B * N; p.L = N; p.nb = w.nb; p.K = K; p.bias_scale = 1.f;
        p.H = H; p.PB = l.PB; p.Dh = l.Dh;
        p.batch_rows = N; p.nbatch = B;
        return p;
    };
    if (stages & KFH_STAGE_IN) {
        if (launch_rows_norm(x, io_dtype, ln, ln + C, xn, rows, C, 1, eps, stream, ending ? N : 0)) return -2;
        LinearArgs p = base(xn, C, C);
        p.nblk = l.nhb; p.Nout = C; p.epi = EPI_FRAG_CH;
        p.W = blob + l.wq; p.out = ws + w.qf;
        if (launch_linear(p, stream)) return -3;
        p.W = blob + l.wk; p.out = ws + w.kf;
        if (launch_linear(p, stream)) return -3;
        p.W = blob + l.wg; p.out = ws + w.gf; p.sigmoid = 1;
        if (launch_linear(p, stream)) return -3;
        p.sigmoid = 0; p.epi = EPI_FRAG_POS;
        p.W = blob + l.wv; p.out = ws + w.vf;
        if (launch_linear(p, stream)) return -3;
        // pair bias: [element][position (a, b)][head] -> tiles indexed (element, head, query a, key b)
        if (rows > 0x7fffffffLL) return -3;
        LinearArgs pb{};
        pb.A = xn; pb.lda = C; pb.rows_a = 1; pb.L = (int)rows; pb.nb = (int)((rows + 31) / 32); pb.K = C;
        pb.W = blob + l.wb; pb.nblk = 1; pb.Nout = H; pb.bias_scale = 1.f; pb.H = 1; pb.PB = 1; pb.Dh = 32;
        pb.out = ws + w.bias; pb.out_dtype = KFH_BF16; pb.ldo = H; pb.epi = EPI_STORE;
        if (launch_linear(pb, stream)) return -3;
        launch_bias_tiles(ws + w.bias, KFH_BF16, reinterpret_cast<uint16_t*>(ws + w.tiles), B, H, N, w.nb, stream,
                          1, (long long)N * H, H, 0, (long long)N * N * H);
        launch_key_codes(mask, reinterpret_cast<uint8_t*>(ws + w.codes), B * N, N, w.nb * 32, ending ? 1 : N, stream,
                         ending ? N : 1, N, (long long)N * N);
    }
    if (stages & KFH_STAGE_CORE) {
        for (int b = 0; b < B; ++b) {
            FlashArgs fa{};
            fa.qf = ws + w.qf + b * w.frag1; fa.kf = ws + w.kf + b * w.frag1; fa.vf = ws + w.vf + b * w.frag1;
            fa.gf = ws + w.gf + b * w.frag1; fa.of = ws + w.of + b * w.frag1;
            fa.biast = ws + w.tiles + b * w.tiles1;
            fa.codes = reinterpret_cast<const uint8_t*>(ws + w.codes + b * w.codes1);
            fa.nrows = N; fa.nb = w.nb; fa.H = H; fa.bias_per_row = 0;
            if (launch_flash(fa, 32 * l.PB, stream)) return -4;
        }
    }
    if (stages & KFH_STAGE_OUT) {
        LinearArgs p = base(ws + w.of, 0, l.ko * 16);
        p.a_frag = 1; p.W = blob + l.wo; p.nblk = C / 32; p.Nout = C; p.epi = EPI_RESID;
        p.out_transposed = ending ? 1 : 0;
        if (residual) { p.aux = residual; p.aux_dtype = io_dtype; p.ld_aux = C; }
        p.out = out; p.out_dtype = io_dtype; p.ldo = C;
        if (launch_linear(p, stream)) return -3;
    }
    return 0;
}

}  // namespace kfh
