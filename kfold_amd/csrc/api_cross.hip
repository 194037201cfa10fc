// C ABI: cross attention with pair bias over local windows (the atom transformer's attention).
#include "../../include/kfold_hip.h"

#include <cmath>

#include "api_util.hpp"
#include "kernels.hpp"

using namespace kfh;

#define KFH_TRY(call, what)                                                             \
    do {                                                                                \
        const int rc_ = (call);                                                         \
        if (rc_ != 0) return fail(KFH_EUNSUPPORTED, "%s: shape not built (%d)", what, rc_); \
    } while (0)

namespace {

// parts = 3 (KFH_ARITH_F32): every packed matrix and every bf16 intermediate is stored as its three
// split3 planes, one after the other
struct CrossLayout {
    int C, H, Dh, PB, Cs, kq, nhb, ko, parts;
    size_t wh, wo_bytes, wa;                                        // bytes of one part
    size_t wq, wk, wv, wg, wo;
    size_t adaq_g, adaq_b, adak_g, adak_b, ada_out;                 // packed [C, Cs] weights
    size_t f_bq, f_lnq_g, f_lnq_b, f_lnk_g, f_lnk_b;                // fp32 vectors
    size_t f_sq_g, f_sk_g, f_adaq_gb, f_adak_gb, f_adaout_b, total;
    bool ok;
    CrossLayout(int C_, int H_, int Cs_, int arith = KFH_ARITH_BF16) : C(C_), H(H_), Cs(Cs_) {
        total = 0;
        parts = arith == KFH_ARITH_F32 ? 3 : 1;
        ok = (arith == KFH_ARITH_BF16 || arith == KFH_ARITH_F32) && C > 0 && H > 0 && C % H == 0 && C % 32 == 0 &&
             C <= 2048 && (Cs == 0 || (Cs % 16 == 0 && Cs <= 2048));
        if (!ok) return;
        Dh = C / H;
        PB = (Dh + 31) / 32;
        ok = PB <= 2;
        if (!ok) return;
        kq = C / 16; nhb = H * PB; ko = nhb * 2;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        wh = (size_t)nhb * kq * 1024;
        wq = take(parts * wh); wk = take(parts * wh); wv = take(parts * wh); wg = take(parts * wh);
        wo_bytes = (size_t)(C / 32) * ko * 1024;
        wo = take(parts * wo_bytes);
        wa = Cs ? (size_t)(C / 32) * (Cs / 16) * 1024 : 0;
        adaq_g = take(parts * wa); adaq_b = take(parts * wa); adak_g = take(parts * wa); adak_b = take(parts * wa);
        ada_out = take(parts * wa);
        f_bq = take(C * 4); f_lnq_g = take(C * 4); f_lnq_b = take(C * 4); f_lnk_g = take(C * 4); f_lnk_b = take(C * 4);
        f_sq_g = take(Cs * 4); f_sk_g = take(Cs * 4); f_adaq_gb = take(C * 4); f_adak_gb = take(C * 4);
        f_adaout_b = take(C * 4);
        total = off;
    }
};

struct CrossWs {
    size_t xq, xk, an, sn, sraw, gate_out, qf, gf, of, kf, vf, tiles, codes, total;
    size_t fq, fk;                     // bytes of one part of a query-side / key-side fragment buffer
    int nbq, nbk;
    CrossWs(const CrossLayout& l, int W, int Lq, int Lk) {
        nbq = (Lq + 31) / 32; nbk = (Lk + 31) / 32;
        size_t off = 0;
        auto take = [&](size_t bytes) { size_t o = off; off += align_up(bytes); return o; };
        const size_t rq = (size_t)W * Lq, rk = (size_t)W * Lk, rmax = rq > rk ? rq : rk;
        const size_t P = l.parts;
        xq = take(P * rq * l.C * 2);
        xk = take(P * rk * l.C * 2);
        an = take(l.Cs ? P * rmax * l.C * 2 : 0);        // LN(a) of the side being conditioned
        sn = take(l.Cs ? P * rmax * l.Cs * 2 : 0);
        sraw = take(l.Cs ? P * rq * l.Cs * 2 : 0);
        gate_out = take(l.Cs ? rq * l.C * (P == 3 ? 4 : 2) : 0);       // fp32 gate in fp32 arithmetic
        fq = (size_t)W * l.H * nbq * l.PB * 2048;
        fk = (size_t)W * l.H * nbk * l.PB * 2048;
        qf = take(P * fq); gf = take(P * fq); of = take(P * fq); kf = take(P * fk); vf = take(P * fk);
        tiles = take((size_t)W * l.H * nbq * nbk * (P == 3 ? kBiasTileF32Bytes : 2048));
        codes = take((size_t)W * nbk * 32);
        total = off;
    }
};

LinearArgs plain(const void* A, long long lda, long long M, int K, const void* W, int Nout) {
    LinearArgs p{};
    p.A = A; p.lda = lda; p.rows_a = 1; p.L = (int)M; p.nb = (int)((M + 31) / 32); p.K = K;
    p.W = W; p.nblk = (Nout + 31) / 32; p.Nout = Nout; p.bias_scale = 1.f;
    p.H = 1; p.PB = 1; p.Dh = 32;
    return p;
}

}  // namespace

extern "C" {

size_t kfh_cross_apb_packed_bytes(int C, int H, int Cs, int arith) { return CrossLayout(C, H, Cs, arith).total; }

int kfh_cross_apb_pack(const void* lnq_w, const void* lnq_b, const void* lnk_w, const void* lnk_b,
                       const void* q_w, const void* q_b, const void* k_w, const void* v_w, const void* g_w,
                       const void* o_w, const void* adaq_s_w, const void* adaq_g_w, const void* adaq_g_b,
                       const void* adaq_bias_w, const void* adak_s_w, const void* adak_g_w,
                       const void* adak_g_b, const void* adak_bias_w, const void* ada_out_w,
                       const void* ada_out_b, int w_dtype, int C, int H, int Cs, int arith, void* blob,
                       void* stream_) {
    const CrossLayout l(C, H, Cs, arith);
    if (!l.ok)
        return fail(KFH_EUNSUPPORTED, "cross_apb_pack: C=%d H=%d Cs=%d arith=%d not supported (C a multiple of 32, Cs of 16, head dim <= 64)", C, H, Cs, arith);
    if (!dtype_ok(w_dtype)) return fail(KFH_EINVAL, "cross_apb_pack: bad w_dtype %d", w_dtype);
    if (!q_w || !k_w || !v_w || !g_w || !o_w || !blob) return fail(KFH_EINVAL, "cross_apb_pack: null pointer");
    if (Cs && (!adaq_g_w || !adaq_bias_w || !adak_g_w || !adak_bias_w || !ada_out_w))
        return fail(KFH_EINVAL, "cross_apb_pack: conditioned module needs the AdaLN / ada_out weights");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    char* b = static_cast<char*>(blob);
    const float qscale = kLog2e / sqrtf((float)l.Dh);
    const size_t blk = (size_t)l.kq * 1024;
    for (int q = 0; q < l.parts; ++q) {
        const int part = l.parts == 3 ? q : -1;
        for (int h = 0; h < H; ++h)
            for (int pp = 0; pp < l.PB; ++pp) {
                const int rows = l.Dh - 32 * pp < 32 ? l.Dh - 32 * pp : 32;
                const int row0 = h * l.Dh + 32 * pp;
                const size_t o = (size_t)q * l.wh + (size_t)(h * l.PB + pp) * blk;
                launch_pack_blocks(q_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, qscale, b + l.wq + o, stream, 0, part);
                launch_pack_blocks(k_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wk + o, stream, 0, part);
                launch_pack_blocks(v_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wv + o, stream, 0, part);
                launch_pack_blocks(g_w, w_dtype, rows, C, C, row0, 1, ROW_NATURAL, K_NATURAL, 1.f, b + l.wg + o, stream, 0, part);
            }
        launch_pack_blocks(o_w, w_dtype, C, l.ko * 16, C, 0, C / 32, ROW_NATURAL, K_ACC_HEADPAD, 1.f,
                           b + l.wo + (size_t)q * l.wo_bytes, stream, l.Dh | ((2 * l.PB) << 16), part);
    }
    auto f32 = [&](size_t off) { return reinterpret_cast<float*>(b + off); };
    launch_copy_f32(q_b, w_dtype, f32(l.f_bq), C, 0.f, stream);
    launch_copy_f32(lnq_w, w_dtype, f32(l.f_lnq_g), C, 1.f, stream);
    launch_copy_f32(lnq_b, w_dtype, f32(l.f_lnq_b), C, 0.f, stream);
    launch_copy_f32(lnk_w, w_dtype, f32(l.f_lnk_g), C, 1.f, stream);
    launch_copy_f32(lnk_b, w_dtype, f32(l.f_lnk_b), C, 0.f, stream);
    if (Cs) {
        auto packa = [&](const void* w, size_t off) {
            for (int q = 0; q < l.parts; ++q)
                launch_pack_blocks(w, w_dtype, C, Cs, Cs, 0, C / 32, ROW_NATURAL, K_NATURAL, 1.f,
                                   b + off + (size_t)q * l.wa, stream, 0, l.parts == 3 ? q : -1);
        };
        packa(adaq_g_w, l.adaq_g); packa(adaq_bias_w, l.adaq_b);
        packa(adak_g_w, l.adak_g); packa(adak_bias_w, l.adak_b);
        packa(ada_out_w, l.ada_out);
        launch_copy_f32(adaq_s_w, w_dtype, f32(l.f_sq_g), Cs, 1.f, stream);
        launch_copy_f32(adak_s_w, w_dtype, f32(l.f_sk_g), Cs, 1.f, stream);
        launch_copy_f32(adaq_g_b, w_dtype, f32(l.f_adaq_gb), C, 0.f, stream);
        launch_copy_f32(adak_g_b, w_dtype, f32(l.f_adak_gb), C, 0.f, stream);
        launch_copy_f32(ada_out_b, w_dtype, f32(l.f_adaout_b), C, 0.f, stream);
    }
    return check_launch("cross_apb_pack");
}

size_t kfh_cross_apb_workspace_bytes(int W, int Lq, int Lk, int C, int H, int Cs, int arith) {
    const CrossLayout l(C, H, Cs, arith);
    if (!l.ok || W <= 0 || Lq <= 0 || Lk <= 0 || Lq > 8192 || Lk > 8192) return 0;
    return CrossWs(l, W, Lq, Lk).total;
}

int kfh_cross_apb_forward(const void* a_q, const void* a_k, const void* s_q, const void* s_k,
                          const void* pair_bias, int bias_dtype, const uint8_t* mask, const void* blob,
                          const void* residual, void* out, void* workspace, size_t workspace_bytes, int W,
                          int Lq, int Lk, int C, int H, int Cs, int apply_norm, float eps, int io_dtype,
                          int arith, void* stream_) {
    const CrossLayout l(C, H, Cs, arith);
    if (!l.ok) return fail(KFH_EUNSUPPORTED, "cross_apb_forward: C=%d H=%d Cs=%d arith=%d not supported", C, H, Cs, arith);
    if (W <= 0 || Lq <= 0 || Lk <= 0) return fail(KFH_EINVAL, "cross_apb_forward: bad shape W=%d Lq=%d Lk=%d", W, Lq, Lk);
    if (Lq > 8192 || Lk > 8192) return fail(KFH_EUNSUPPORTED, "cross_apb_forward: window of %d x %d", Lq, Lk);
    if (!dtype_ok(io_dtype) || !dtype_ok(bias_dtype)) return fail(KFH_EINVAL, "cross_apb_forward: bad dtype");
    if (!a_q || !a_k || !pair_bias || !mask || !blob || !out || !workspace)
        return fail(KFH_EINVAL, "cross_apb_forward: null pointer argument");
    const bool cond = Cs > 0 && apply_norm;
    if (cond && (!s_q || !s_k)) return fail(KFH_EINVAL, "cross_apb_forward: conditioned module needs s_q and s_k");
    const CrossWs w(l, W, Lq, Lk);
    if (workspace_bytes < w.total)
        return fail(KFH_EINVAL, "cross_apb_forward: workspace %zu < %zu bytes", workspace_bytes, w.total);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* b = static_cast<const char*>(blob);
    char* ws = static_cast<char*>(workspace);
    auto f32p = [&](size_t off) { return reinterpret_cast<const float*>(b + off); };
    const long long rq = (long long)W * Lq, rk = (long long)W * Lk;
    uint16_t* xq = reinterpret_cast<uint16_t*>(ws + w.xq);
    uint16_t* xk = reinterpret_cast<uint16_t*>(ws + w.xk);

    const int P = l.parts;
    // with P = 3 a [rows, ch] bf16 tensor is three planes `rows * ch * 2` bytes apart (split3)
    auto plane = [&](long long r, int ch) { return P == 3 ? (size_t)r * ch * 2 : (size_t)0; };

    // 1. normalised rows of both sides (LayerNorm, or AdaLN with the side's own conditioning)
    if (!apply_norm) {
        KFH_TRY(launch_rows_norm(a_q, io_dtype, nullptr, nullptr, xq, rq, C, 0, eps, stream, 0, P), "rows_norm");
        KFH_TRY(launch_rows_norm(a_k, io_dtype, nullptr, nullptr, xk, rk, C, 0, eps, stream, 0, P), "rows_norm");
    } else if (!Cs) {
        KFH_TRY(launch_rows_norm(a_q, io_dtype, f32p(l.f_lnq_g), f32p(l.f_lnq_b), xq, rq, C, 1, eps, stream, 0, P), "rows_norm");
        KFH_TRY(launch_rows_norm(a_k, io_dtype, f32p(l.f_lnk_g), f32p(l.f_lnk_b), xk, rk, C, 1, eps, stream, 0, P), "rows_norm");
    } else {
        uint16_t* an = reinterpret_cast<uint16_t*>(ws + w.an);
        uint16_t* sn = reinterpret_cast<uint16_t*>(ws + w.sn);
        auto adaln = [&](const void* a, const void* s, long long rows, size_t f_s_g, size_t w_g, size_t w_b,
                         size_t f_gb, uint16_t* dst) -> int {
            if (launch_rows_norm(a, io_dtype, nullptr, nullptr, an, rows, C, 1, eps, stream, 0, P)) return -2;
            if (launch_rows_norm(s, io_dtype, f32p(f_s_g), nullptr, sn, rows, Cs, 1, eps, stream, 0, P)) return -2;
            LinearArgs p = plain(sn, Cs, rows, Cs, b + w_g, C);
            p.W2 = b + w_b; p.bias = f32p(f_gb);
            p.aux = an; p.aux_dtype = KFH_BF16; p.ld_aux = C;
            p.out = dst; p.out_dtype = KFH_BF16; p.ldo = C; p.epi = EPI_ADALN;
            p.parts = P; p.a_part = plane(rows, Cs); p.w_part = l.wa; p.aux_part = plane(rows, C);
            p.out_part = plane(rows, C);
            return launch_linear(p, stream);
        };
        KFH_TRY(adaln(a_q, s_q, rq, l.f_sq_g, l.adaq_g, l.adaq_b, l.f_adaq_gb, xq), "adaln (query side)");
        KFH_TRY(adaln(a_k, s_k, rk, l.f_sk_g, l.adak_g, l.adak_b, l.f_adak_gb, xk), "adaln (key side)");
        // output gate sigmoid(W_ada s_q + b_ada) on the raw query-side conditioning
        uint16_t* sraw = reinterpret_cast<uint16_t*>(ws + w.sraw);
        KFH_TRY(launch_rows_norm(s_q, io_dtype, nullptr, nullptr, sraw, rq, Cs, 0, eps, stream, 0, P), "rows_norm");
        LinearArgs g = plain(sraw, Cs, rq, Cs, b + l.ada_out, C);
        g.bias = f32p(l.f_adaout_b);
        g.out = ws + w.gate_out; g.out_dtype = P == 3 ? KFH_F32 : KFH_BF16; g.ldo = C; g.epi = EPI_SIGMOID;
        g.parts = P; g.a_part = plane(rq, Cs); g.w_part = l.wa;
        KFH_TRY(launch_linear(g, stream), "linear");
    }

    // 2. projections into fragment order: q (bias, pre-scaled), gate from the query side; k, v
    //    from the key side.  "Rows" of the attention are the windows.
    {
        LinearArgs p = plain(xq, C, Lq, C, nullptr, C);
        p.rows_a = W; p.nb = w.nbq; p.nblk = l.nhb; p.H = H; p.PB = l.PB; p.Dh = l.Dh;
        p.parts = P; p.a_part = plane(rq, C); p.w_part = l.wh; p.out_part = w.fq;
        p.epi = EPI_FRAG_CH;
        p.W = b + l.wq; p.bias = f32p(l.f_bq); p.bias_scale = kLog2e / sqrtf((float)l.Dh);
        p.out = ws + w.qf;
        KFH_TRY(launch_linear(p, stream), "linear");
        p.bias = nullptr;
        p.W = b + l.wg; p.out = ws + w.gf; p.sigmoid = 1;
        KFH_TRY(launch_linear(p, stream), "linear");
        LinearArgs k = plain(xk, C, Lk, C, b + l.wk, C);
        k.rows_a = W; k.nb = w.nbk; k.nblk = l.nhb; k.H = H; k.PB = l.PB; k.Dh = l.Dh;
        k.parts = P; k.a_part = plane(rk, C); k.w_part = l.wh; k.out_part = w.fk;
        k.epi = EPI_FRAG_CH; k.out = ws + w.kf;
        KFH_TRY(launch_linear(k, stream), "linear");
        k.epi = EPI_FRAG_POS; k.W = b + l.wv; k.out = ws + w.vf;
        KFH_TRY(launch_linear(k, stream), "linear");
    }

    // 3. bias tiles (one batch per window), key codes, attention
    if (P == 3)
        launch_bias_tiles_f32(pair_bias, bias_dtype, reinterpret_cast<float*>(ws + w.tiles), W, H, Lq, w.nbq, stream, Lk);
    else
        launch_bias_tiles(pair_bias, bias_dtype, reinterpret_cast<uint16_t*>(ws + w.tiles), W, H, Lq, w.nbq, stream,
                          0, 0, 0, Lk);
    uint8_t* codes = reinterpret_cast<uint8_t*>(ws + w.codes);
    launch_key_codes(mask, codes, W, Lk, w.nbk * 32, Lk, stream);
    FlashArgs fa{};
    fa.qf = ws + w.qf; fa.kf = ws + w.kf; fa.vf = ws + w.vf; fa.gf = ws + w.gf; fa.of = ws + w.of;
    fa.biast = ws + w.tiles; fa.codes = codes;
    fa.nrows = W; fa.nb = w.nbk; fa.nbq = w.nbq; fa.H = H; fa.bias_per_row = 1;
    if (P == 3) {
        fa.q_part = fa.g_part = fa.o_part = w.fq;
        fa.k_part = fa.v_part = w.fk;
        if (launch_flash_split(fa, 32 * l.PB, stream) != 0) return fail(KFH_EUNSUPPORTED, "cross_apb_forward: attention shape");
    } else if (launch_flash(fa, 32 * l.PB, stream) != 0) {
        return fail(KFH_EUNSUPPORTED, "cross_apb_forward: attention shape");
    }

    // 4. output projection (+ conditioning gate, + residual)
    {
        LinearArgs p{};
        p.A = ws + w.of; p.a_frag = 1; p.rows_a = W; p.L = Lq; p.nb = w.nbq; p.K = l.ko * 16;
        p.W = b + l.wo; p.nblk = C / 32; p.Nout = C; p.bias_scale = 1.f;
        p.H = H; p.PB = l.PB; p.Dh = l.Dh;
        p.parts = P; p.a_part = w.fq; p.w_part = l.wo_bytes;
        p.epi = EPI_RESID;
        if (cond) {
            p.gate = reinterpret_cast<const uint16_t*>(ws + w.gate_out); p.ld_gate = C;
            p.gate_dtype = P == 3 ? KFH_F32 : KFH_BF16;
        }
        if (residual) { p.aux = residual; p.aux_dtype = io_dtype; p.ld_aux = C; }
        p.out = out; p.out_dtype = io_dtype; p.ldo = C;
        KFH_TRY(launch_linear(p, stream), "linear");
    }
    return check_launch("cross_apb_forward");
}

}  // extern "C"
