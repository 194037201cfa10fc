// Internal launch interface between the C-ABI layer (api.hip) and the kernel files.
#pragma once
#include "common.hpp"

namespace kfh {

// ---- weight packing (pack.hip) ----------------------------------------------------------
enum : int { ROW_NATURAL = 0, ROW_INTERLEAVE2 = 1, ROW_INTERLEAVE4 = 2 };
enum : int { K_NATURAL = 0, K_ACC = 1, K_HALF = 2 };

constexpr size_t kBlockBytes = 32 * kC * 2;   // one packed 32-row x 128-channel block = 8 KiB

void launch_pack_blocks(const void* src, int wdtype, int src_rows, int K, int ld, int row0,
                        int nblk, int row_mode, int k_mode, float scale, void* dst,
                        hipStream_t stream);
void launch_copy_f32(const void* src, int wdtype, float* dst, int n, float fill,
                     hipStream_t stream);

// ---- triangle multiplication (trimul.hip, contract.hip) ------------------------------------
// Packed weight blob of one triangle-multiplication module (C = D = 128):
//   [0, 128K)     8 steps x { p_in block cb, g_in block cb }   (32 channels of a|b each)
//   [128K, 160K)  2 steps x { g_out blocks 2s, 2s+1 }          (ROW_INTERLEAVE2)
//   [160K, 192K)  p_out, 4 blocks                               (ROW_INTERLEAVE4, K_HALF)
//   [192K, +2K)   fp32: ln_in gamma, ln_in beta, ln_out gamma, ln_out beta (128 each)
constexpr size_t kTmInOff = 0;
constexpr size_t kTmGateOff = 16 * kBlockBytes;
constexpr size_t kTmOutOff = 20 * kBlockBytes;
constexpr size_t kTmLnOff = 24 * kBlockBytes;
constexpr size_t kTmBlobBytes = kTmLnOff + 4 * kC * sizeof(float);

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }
// side of the zero-padded square planes the contraction runs on
inline int trimul_np(int N) { return round_up(N, 128); }

void launch_trimul_in(const void* z, int io_dtype, const uint8_t* mask, const char* blob,
                      uint16_t* planes, uint16_t* gate, int N, int Np, int incoming, float eps,
                      hipStream_t stream);
void launch_contract(const uint16_t* planes_a, const uint16_t* planes_b, uint16_t* planes_y,
                     int Np, int D, hipStream_t stream);
void launch_trimul_out(const uint16_t* planes_y, const uint16_t* gate, const char* blob,
                       const void* residual, void* out, int io_dtype, int N, int Np, float eps,
                       hipStream_t stream);

// ---- triangle attention (triattn.hip) ------------------------------------------------------
// Packed weight blob of one triangle-attention module (C = 128, 4 heads x 32):
//   [0, 144K)     9 steps x 2 blocks: {q_h,k_h} h=0..3, {g_h,v_h} h=0..3, {pair bias, zero};
//                 q and the pair bias are pre-multiplied by log2(e) (and q by 1/sqrt(32))
//   [144K, 176K)  o projection, 4 blocks (ROW_INTERLEAVE4, K_ACC)
//   [176K, +1K)   fp32: LN gamma, beta
constexpr size_t kTaProjOff = 0;
constexpr size_t kTaOutOff = 18 * kBlockBytes;
constexpr size_t kTaLnOff = 22 * kBlockBytes;
constexpr size_t kTaBlobBytes = kTaLnOff + 2 * kC * sizeof(float);

struct TriattnWorkspace {
    void *qf, *kf, *vf, *gf, *of;   // fragment buffers, N * 4 * nb * 2 KiB each
    float* biasf;                    // 4 * nb * nb tiles of 4 KiB
    uint8_t* codes;                  // N * nb * 32 key codes
};

void launch_fill_zero(void* dst, size_t bytes, hipStream_t stream);
void launch_triattn(const void* x, int io_dtype, const uint8_t* mask, const char* blob,
                    const TriattnWorkspace& ws, const void* residual, void* out, int N, int ending,
                    float eps, hipStream_t stream);

}  // namespace kfh
