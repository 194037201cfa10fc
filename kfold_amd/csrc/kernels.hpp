// Internal launch interface between the C-ABI layer (api.hip) and the kernel files.
#pragma once
#include "common.hpp"

namespace kfh {

// ---- weight packing (pack.hip) ----------------------------------------------------------
enum : int { ROW_NATURAL = 0, ROW_INTERLEAVE2 = 1, ROW_INTERLEAVE4 = 2 };
enum : int { K_NATURAL = 0, K_ACC = 1, K_HALF = 2, K_ACC_HEADPAD = 3 };

constexpr size_t kBlockBytes = 32 * kC * 2;   // one packed 32-row x 128-channel block = 8 KiB

// K: number of k-slots (padded contraction length); ld: row pitch of src in elements
// part: -1 packs bf16(scale * w); 0..2 packs that part of split3(scale * w) (fp32 arithmetic)
void launch_pack_blocks(const void* src, int wdtype, int src_rows, int K, int ld, int row0,
                        int nblk, int row_mode, int k_mode, float scale, void* dst,
                        hipStream_t stream, int kparam = 0, int part = -1);
void launch_copy_f32(const void* src, int wdtype, float* dst, int n, float fill,
                     hipStream_t stream);

// ---- triangle multiplication (trimul.hip, contract.hip) ------------------------------------
// Packed weight blob of one triangle-multiplication module (C = D = 128):
//   [0, 32K)      g_out, 4 blocks                               (ROW_INTERLEAVE4), output phase
//   [32K, 160K)   8 steps x { p_in block cb, g_in block cb }   (32 channels of a|b each)
//                 all gate weights (g_out, g_in) are pre-multiplied by -log2(e)
//   [160K, 192K)  p_out, 4 blocks                               (ROW_INTERLEAVE4, K_HALF)
//   [192K, +2K)   fp32: ln_in gamma, ln_in beta, ln_out gamma, ln_out beta (128 each)
constexpr size_t kTmGateOff = 0;
constexpr size_t kTmAbOff = 4 * kBlockBytes;
constexpr size_t kTmOutOff = 20 * kBlockBytes;
constexpr size_t kTmLnOff = 24 * kBlockBytes;
constexpr size_t kTmBlobBytes = kTmLnOff + 4 * kC * sizeof(float);

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }
// side of the zero-padded square planes the contraction runs on
inline int trimul_np(int N) { return round_up(N, 128); }

void launch_trimul_in(const void* z, int io_dtype, const uint8_t* mask, const char* blob,
                      uint16_t* planes, int N, int Np, int incoming, float eps, hipStream_t stream);
// rows of one contraction tile at this plane size: a range of result rows handed to
// launch_contract starts at a multiple of it
inline int contract_tile_rows(int Np) { return Np % 256 == 0 ? 256 : 128; }
// row0 / nrows: only the result rows [row0, row0 + nrows) of every plane (nrows < 0: all Np rows);
// the same kernels on offset pointers, so a result computed in ranges has the bits of one launch
void launch_contract(const uint16_t* planes_a, const uint16_t* planes_b, uint16_t* planes_y,
                     int Np, int D, hipStream_t stream, int row0 = 0, int nrows = -1);
void launch_trimul_out(const uint16_t* planes_y, const void* z, const char* blob,
                       const void* residual, void* out, int io_dtype, int N, int Np, float eps,
                       hipStream_t stream, int row0 = 0, int nrows = -1);

// any other width that is a multiple of 32 (trimul_generic.hip), from the token-track kernels
size_t trimul_generic_blob_bytes(int C);
size_t trimul_generic_ws_bytes(int N, int C, int B = 1);
int trimul_generic_pack(const void* ln_in_w, const void* ln_in_b, const void* p_in_w, const void* g_in_w,
                        const void* ln_out_w, const void* ln_out_b, const void* p_out_w, const void* g_out_w,
                        int w_dtype, int C, void* blob, hipStream_t stream);
// B batch elements at once (ws of trimul_generic_ws_bytes(N, C, B))
int trimul_generic_forward(const void* z, int io_dtype, const uint8_t* mask, const char* blob, char* ws,
                           const void* residual, void* out, int B, int N, int C, int incoming, float eps,
                           int stages, hipStream_t stream);

// other pair widths (trimul_wide.hip; C = 256): same interface, blob layout in that file
size_t trimul_wide_blob_bytes(int C);
void trimul_wide_offsets(int C, size_t* gate, size_t* ab, size_t* out, size_t* ln, size_t* blk);
int launch_trimul_in_wide(const void* z, int io_dtype, const uint8_t* mask, const char* blob, uint16_t* planes,
                          int N, int Np, int C, int incoming, float eps, hipStream_t stream);
int launch_trimul_out_wide(const uint16_t* planes_y, const void* z, const char* blob, const void* residual,
                           void* out, int io_dtype, int N, int Np, int C, float eps, hipStream_t stream,
                           int row0 = 0, int nrows = -1);

// ---- triangle attention (triattn.hip) ------------------------------------------------------
// Packed weight blob of one triangle-attention module (C = 128, 4 heads x 32):
//   [0, 112K)     7 steps x 2 blocks: {q_h,k_h} h=0..3, {v_0,v_1}, {v_2,v_3}, {pair bias, zero};
//                 q and the pair bias are pre-multiplied by log2(e) (and q by 1/sqrt(32))
//   [112K, 144K)  gate g_h, 4 blocks, pre-multiplied by -log2(e) (output phase)
//   [144K, 176K)  o projection, 4 blocks (ROW_INTERLEAVE4, K_ACC)
//   [176K, +1K)   fp32: LN gamma, beta
constexpr size_t kTaProjOff = 0;
constexpr size_t kTaGateOff = 14 * kBlockBytes;
constexpr size_t kTaOutOff = 18 * kBlockBytes;
constexpr size_t kTaLnOff = 22 * kBlockBytes;
constexpr size_t kTaBlobBytes = kTaLnOff + 2 * kC * sizeof(float);

struct TriattnWorkspace {
    void *qf, *kf, *vf, *of;        // fragment buffers, N * 4 * nb * 2 KiB each
    uint16_t* biast;                 // 4 * nb * nb bf16 tiles of 2 KiB
    uint8_t* codes;                  // N * nb * 32 key codes
};

// ---- attention core (flash.hip) --------------------------------------------------------------
struct FlashArgs {
    const void *qf, *kf, *vf, *gf;   // fragment-order operands; gf (the sigmoid gate) may be null
    void* of;                         // gated output fragments
    const void* biast;                // bf16 bias tiles [batch][h][query block][key block] (bias_tile_elem layout)
    const uint8_t* codes;             // [nrows][nb*32] key codes
    int nrows, nb, H;                 // nb: key blocks of 32 per row
    int nbq;                          // query blocks per row (0: same as nb, self attention)
    int bias_per_row;                 // 0: one bias for all rows, 1: bias batch index = row
    int qgroups, nchunks;             // filled in by launch_flash
    int rowranges, rows_per_range;    // strip kernel: rows are split into ranges per workgroup
    // fp32 arithmetic (launch_flash_split only): every fragment operand comes as three bf16 parts
    // (split3), `*_part` bytes apart; the bias tiles are fp32 (bias_tile_f32_elem layout)
    size_t q_part, k_part, v_part, g_part, o_part;
};
// full_rows > 0: args describe a range of the rows of a problem with full_rows rows; the kernel is
// chosen as for the whole problem (returns -3 if the range is too short for that kernel)
int launch_flash(const FlashArgs& args, int head_dim_pad, hipStream_t stream, int full_rows = 0);
// the same attention in fp32 arithmetic on split operands (flash_split.hip)
int launch_flash_split(const FlashArgs& args, int head_dim_pad, hipStream_t stream);

void launch_fill_zero(void* dst, size_t bytes, hipStream_t stream);
// returns 0, or the non-zero status of the attention launch (shape not built, HIP error)
int launch_triattn(const void* x, int io_dtype, const uint8_t* mask, const char* blob,
                    const TriattnWorkspace& ws, const void* residual, void* out, int N, int ending,
                    float eps, int stages, hipStream_t stream, int row0 = 0, int nrows = -1);

// other widths / head shapes (triattn_generic.hip): head dim <= 64, C a multiple of 32
size_t triattn_generic_blob_bytes(int C, int H);
size_t triattn_generic_ws_bytes(int N, int C, int H, int B = 1);
int triattn_generic_pack(const void* ln_w, const void* ln_b, const void* q_w, const void* k_w, const void* v_w,
                         const void* g_w, const void* bias_w, const void* o_w, int w_dtype, int C, int H,
                         void* blob, hipStream_t stream);
// B batch elements at once (ws of triattn_generic_ws_bytes(N, C, H, B)); only the attention core is
// launched per element
int triattn_generic_forward(const void* x, int io_dtype, const uint8_t* mask, const char* blob, char* ws,
                            const void* residual, void* out, int B, int N, int C, int H, int ending, float eps,
                            int stages, hipStream_t stream);

// ---- pair transition (transition.hip) ----------------------------------------------------
// Packed blob (C = 128 or 256, expansion E): C*E/32 steps x { u block, v block, W_out slice of the
// step's 32 hidden channels as C/32 blocks x 2 k-steps (ROW_INTERLEAVE4, K_ACC) } (24 KiB per step
// at C = 128, 48 KiB at C = 256), then fp32 LN gamma, beta.
inline size_t transition_blob_bytes(int E, int C = kC) {
    return (size_t)(C * E / 32) * 3 * 32 * C * 2 + 2 * (size_t)C * sizeof(float);
}
inline bool transition_fused(int C, int E) { return (C == kC || C == 256) && (E == 2 || E == 4); }
int launch_pair_transition(const void* x, int io_dtype, const char* blob, int expansion,
                           const void* residual, const uint8_t* mask, void* out, long long M,
                           float eps, hipStream_t stream);
// the same kernel at C = 256 (transition_wide.hip)
int launch_pair_transition_wide(const void* x, int io_dtype, const char* blob, int expansion,
                                const void* residual, const uint8_t* mask, void* out, long long M,
                                float eps, hipStream_t stream, int C);

// ---- pair bias projection (pairbias.hip): blob = one packed block (heads as rows, scaled by
// log2 e) followed by fp32 LN gamma, beta
constexpr size_t kPbBlobBytes = kBlockBytes + 2 * kC * sizeof(float);
void launch_pair_bias(const void* z, int io_dtype, const char* blob, uint16_t* tiles, int N, int H,
                      float eps, hipStream_t stream);

// ---- Parcae recurrence step (parcae.hip), C = 128 or 256 ------------------------------------
// blob: packed B [C/32 blocks][C/16 k-steps][64][8] bf16 (ROW_INTERLEAVE4 within groups of 128
// output channels), fp32 LN gamma, beta [2C], fp32 a [C], then C*C fp32 of pack-time scratch
inline size_t parcae_blob_bytes(int C) { return (size_t)C * C * 2 + 3 * (size_t)C * 4 + (size_t)C * C * 4; }
void launch_parcae_dynamics(const void* log_a, const void* log_delta, const void* b_cont, int wdtype,
                            float* a_out, float* b_out, int C, hipStream_t stream);
int launch_parcae_step(const void* z, const void* u, const void* u2, int io_dtype, const char* blob, void* out,
                       long long M, int C, float eps, hipStream_t stream);

// ---- single-track helpers (rows.hip, linear.hip) -------------------------------------------
// transpose_n > 0: the M = n*n rows are written transposed as an [n, n] grid of rows
// parts = 3: the result is written as the three split3 planes out[q][M][C] (fp32 arithmetic)
int launch_rows_norm(const void* x, int io_dtype, const float* gamma, const float* beta, uint16_t* out,
                     long long M, int C, int normalize, float eps, hipStream_t stream, int transpose_n = 0,
                     int parts = 1);
// mask element of (row a, key k) is mask[a * mask_stride + k * key_stride]; with rows_per_batch > 0
// row a = b * rows_per_batch + i and the element is mask[b * batch_stride + i * mask_stride + k * key_stride]
void launch_key_codes(const uint8_t* mask, uint8_t* codes, int rows, int L, int Lp,
                      long long mask_stride, hipStream_t stream, long long key_stride = 1,
                      int rows_per_batch = 0, long long batch_stride = 0);
// source element (t = batch*H + head, q, k) at t*st + q*sq + k*sk; all zero = dense [.., H, L, Lk];
// with sb != 0 at batch*sb + head*st + q*sq + k*sk.  L queries in nb blocks, Lk keys (0: = L)
void launch_bias_tiles(const void* dense, int io_dtype, uint16_t* tiles, int nbatch, int H, int L, int nb,
                       hipStream_t stream, long long st = 0, long long sq = 0, long long sk = 0, int Lk = 0,
                       long long sb = 0);
// the same as fp32 tiles of 4 KiB (bias_tile_f32_elem layout) for the fp32 arithmetic
void launch_bias_tiles_f32(const void* dense, int io_dtype, float* tiles, int nbatch, int H, int L, int nb,
                           hipStream_t stream, int Lk = 0);

enum : int { EPI_STORE = 0, EPI_SIGMOID, EPI_SWIGLU, EPI_ADALN, EPI_RESID, EPI_FRAG_CH, EPI_FRAG_POS, EPI_PLANES };

// Rows are addressed as (a, position): a < rows_a, position < L, global row = a * L + position,
// position blocks of 32 (nb = ceil(L / 32)).  Plain [M, K] problems use rows_a = 1, L = M.
struct LinearArgs {
    const void* A; long long lda; int a_frag;    // row-major bf16 [rows][lda] or fragment order
    int a_shared, aux_shared, gate_shared;       // operand has one `a` slice shared by all rows_a
    int rows_a, L, nb, K;                        // K: contraction length in the packed weight
    const void* W; const void* W2; int nblk;     // packed blocks [nblk][K/16][64 lanes][8]
    const float* bias; float bias_scale; int sigmoid;
    const void* aux; int aux_dtype; long long ld_aux;
    const uint16_t* gate; long long ld_gate;
    void* out; int out_dtype; long long ldo; int Nout;
    int epi;
    int H, PB, Dh;                               // heads, 32-blocks per padded head, real head dim
    int out_transposed;                          // EPI_RESID: out / aux row of (a, position) is position * rows_a + a
                                                 // (inside each batch element of batch_rows row groups, see below)
    // fp32 arithmetic: parts = 3 — A, W, W2 and every bf16 output (row-major or fragments) are three
    // split3 planes, `*_part` bytes apart; the EPI_ADALN aux is summed over its three planes;
    // gate_dtype says how the EPI_RESID gate is stored (a KFH_F32 gate in this mode)
    int parts;
    size_t a_part, w_part, out_part, aux_part;
    int gate_dtype;
    // EPI_PLANES: out is bf16 channel-major planes [Nout][ldo][ldo], value (acc * sigmoid(acc2)) or 0
    // where the position's mask byte is 0, stored at plane[c][a * ldo + position]; the mask byte of
    // (a, position) is mask[a * L + position], or mask[position * rows_a + a] with mask_transposed.
    // EPI_RESID: optional mask byte per output row (0 zeroes the row)
    const uint8_t* mask; int mask_transposed;
    // A batch folded into the row groups: a = b * batch_rows + i (batch_rows = 0: one element, i = a).
    // Transposed indices (out_transposed, mask_transposed) are taken inside an element:
    // b * batch_rows * L + position * batch_rows + i.  EPI_PLANES with nbatch > 1 stores channel c of
    // element b at plane (c / plane_side) * nbatch * plane_side + b * plane_side + c % plane_side, row i.
    int batch_rows, nbatch, plane_side;
};
int launch_linear(const LinearArgs& p, hipStream_t stream);

}  // namespace kfh
