// Host-side execution model for the kernel sources of kfold_amd/csrc — TEST INFRASTRUCTURE.
//
// The parity suite's CPU leg compiles the very same .hip files as ordinary C++ for x86-64 with
// this header on the include path in place of HIP's.  A kernel launch then runs on the host:
// every workgroup in turn (several at once on a thread pool), every lane of it as a fiber, with
// the operations that couple lanes (MFMA, shuffles, ballots, barriers) implemented as
// rendezvous points of the wavefront or workgroup.  "Device" pointers are host pointers.
//
// What this checks: the index arithmetic, the data layouts, the MFMA operand conventions, the
// control flow and the numerics of the kernels, and — with the guard-paged allocator of
// hostsim.cpp — that no lane touches memory outside its buffers.  What it cannot check: timing,
// occupancy, memory-ordering hazards between lanes of one wavefront that real hardware resolves
// by running them in lock step (lanes run one after another between two rendezvous points here).
//
// Nothing in the product loads this build; it never runs on a GPU box's device.
#pragma once
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>

// ---- language extensions -------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static thread_local
#define __align__(n) __attribute__((aligned(n)))
#define HOSTSIM 1

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
constexpr int hipFuncAttributeMaxDynamicSharedMemorySize = 8;
constexpr int hipDeviceAttributeMultiprocessorCount = 63;
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "host simulation"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, int, int) { return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = 256; return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
template <class T> inline hipError_t hipGetSymbolAddress(void** p, T* sym) { *p = (void*)sym; return hipSuccess; }

namespace hostsim {

typedef __attribute__((ext_vector_type(8))) __bf16 v8bf;
typedef __attribute__((ext_vector_type(16))) float v16f;
typedef __attribute__((ext_vector_type(2))) uint32_t v2u;

struct Wave;
struct Block;
struct Lane {
    dim3 tidx, bidx, bdim, gdim;
    int lane;            // 0..63 inside the wavefront
    Wave* wave;
    Block* block;
    void* fiber;
};
Lane* cur();             // lane running on this OS thread

// Wavefront rendezvous: every live lane of the wavefront deposits a pointer to its arguments;
// the last one to arrive runs `fn(slots, mask)` once for all (slots[l] is null for lanes that
// have exited), then everybody continues.  `tag` names the operation: lanes of one wavefront
// meeting in different operations is a divergence bug and aborts with a report.
typedef void (*Thunk)(void* fnobj, void** slots, unsigned long long mask);
void wave_rendezvous(int tag, void* mine, Thunk thunk, void* fnobj);
void block_barrier();
char* dynamic_lds();

template <class A, class F>
inline void collective(int tag, A* mine, F& fn) {
    wave_rendezvous(tag, mine,
                    [](void* f, void** s, unsigned long long m) { (*static_cast<F*>(f))(reinterpret_cast<A**>(s), m); },
                    &fn);
}

void launch(const char* name, dim3 grid, dim3 block, size_t dyn_lds, const std::function<void()>& body);

// ---- cross-lane operations -------------------------------------------------------------------
struct ShflArgs { uint32_t v, r; int src; };
inline uint32_t shfl_bits(uint32_t v, int src_lane) {
    ShflArgs a{v, v, src_lane};
    auto fn = [](ShflArgs** s, unsigned long long) {
        uint32_t vals[64];
        for (int l = 0; l < 64; ++l) vals[l] = s[l] ? s[l]->v : 0u;
        for (int l = 0; l < 64; ++l)
            if (s[l]) s[l]->r = s[s[l]->src & 63] ? vals[s[l]->src & 63] : vals[l];
    };
    collective(1, &a, fn);
    return a.r;
}

struct BallotArgs { int pred; unsigned long long r; };
inline unsigned long long ballot(int pred) {
    BallotArgs a{pred, 0ull};
    auto fn = [](BallotArgs** s, unsigned long long) {
        unsigned long long m = 0;
        for (int l = 0; l < 64; ++l) if (s[l] && s[l]->pred) m |= 1ull << l;
        for (int l = 0; l < 64; ++l) if (s[l]) s[l]->r = m;
    };
    collective(2, &a, fn);
    return a.r;
}

struct FirstArgs { int v, r; };
inline int readfirstlane(int v) {
    FirstArgs a{v, v};
    auto fn = [](FirstArgs** s, unsigned long long) {
        int first = 0;
        for (int l = 0; l < 64; ++l) if (s[l]) { first = s[l]->v; break; }
        for (int l = 0; l < 64; ++l) if (s[l]) s[l]->r = first;
    };
    collective(3, &a, fn);
    return a.r;
}

// v_permlane32_swap: the upper 32 lanes of the first operand trade places with the lower 32
// lanes of the second; returns {first, second} afterwards.
struct SwapArgs { uint32_t a, b, ra, rb; };
inline v2u permlane32_swap(uint32_t a_, uint32_t b_) {
    SwapArgs a{a_, b_, a_, b_};
    auto fn = [](SwapArgs** s, unsigned long long) {
        for (int l = 0; l < 32; ++l) {
            if (!s[l] || !s[l + 32]) continue;
            const uint32_t hi_a = s[l + 32]->a, lo_b = s[l]->b;
            s[l + 32]->ra = lo_b;
            s[l]->rb = hi_a;
        }
    };
    collective(4, &a, fn);
    return v2u{a.ra, a.rb};
}

inline void wave_barrier() {
    int dummy = 0;
    auto fn = [](int**, unsigned long long) {};
    collective(5, &dummy, fn);
}

// v_mfma_f32_32x32x16_bf16, D = C + A[32x16] B[16x32]:
//   A: lane l holds A[l % 32][8 * (l / 32) + 0..7];  B: lane l holds B[8 * (l / 32) + 0..7][l % 32]
//   C/D: lane l holds D[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32], v = 0..15
struct MfmaArgs { v8bf a, b; v16f c; };
void mfma_32x32x16_bf16_all(MfmaArgs** s);     // hostsim.cpp
inline v16f mfma_32x32x16_bf16(v8bf a, v8bf b, v16f c) {
    MfmaArgs args{a, b, c};
    auto fn = [](MfmaArgs** s, unsigned long long) { mfma_32x32x16_bf16_all(s); };
    collective(6, &args, fn);
    return args.c;
}

}  // namespace hostsim

// ---- what kernel code sees --------------------------------------------------------------------
#define threadIdx (::hostsim::cur()->tidx)
#define blockIdx (::hostsim::cur()->bidx)
#define blockDim (::hostsim::cur()->bdim)
#define gridDim (::hostsim::cur()->gdim)

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    ::hostsim::launch(#kernel, dim3(grid), dim3(block), (size_t)(shmem), [=]() { kernel(__VA_ARGS__); })

// dynamic LDS: `extern __shared__ T name[];` is spelled HIP_DYNAMIC_SHARED(T, name) in the sources
#define HIP_DYNAMIC_SHARED(type, var) type* var = reinterpret_cast<type*>(::hostsim::dynamic_lds());

inline void __syncthreads() { ::hostsim::block_barrier(); }
inline float __shfl_xor(float v, int mask) {
    uint32_t u;
    memcpy(&u, &v, 4);
    u = ::hostsim::shfl_bits(u, ::hostsim::cur()->lane ^ mask);
    memcpy(&v, &u, 4);
    return v;
}
inline int __shfl_xor(int v, int mask) {
    return (int)::hostsim::shfl_bits((uint32_t)v, ::hostsim::cur()->lane ^ mask);
}
inline unsigned long long __ballot(int pred) { return ::hostsim::ballot(pred); }
inline int __any(int pred) { return ::hostsim::ballot(pred) != 0ull; }
inline int __popc(unsigned v) { return __builtin_popcount(v); }
inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline int min(int a, int b) { return a < b ? a : b; }
inline int max(int a, int b) { return a > b ? a : b; }
inline long long min(long long a, long long b) { return a < b ? a : b; }
inline long long max(long long a, long long b) { return a > b ? a : b; }
inline size_t min(size_t a, size_t b) { return a < b ? a : b; }
inline size_t max(size_t a, size_t b) { return a > b ? a : b; }

#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) ::hostsim::mfma_32x32x16_bf16((a), (b), (c))
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) ::hostsim::permlane32_swap((a), (b))
#define __builtin_amdgcn_readfirstlane(v) ::hostsim::readfirstlane((v))
#define __builtin_amdgcn_wave_barrier() ::hostsim::wave_barrier()
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_rsqf(x) (1.0f / sqrtf((x)))
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_exp2f(x) exp2f((x))
