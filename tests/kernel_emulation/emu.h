// A lane-accurate host execution of one workgroup of a gfx950 kernel, for tests (TEST INFRASTRUCTURE ONLY).
//
// Every lane is a fibre running the kernel's own source as scalar code. Fibres meet where the hardware makes lanes
// meet: at matrix instructions, LDS transpose reads and lane permutes (the 64 lanes of a wavefront exchange
// operands), at wave barriers, and at workgroup barriers. Between those points a fibre runs alone, wavefront after
// wavefront in an order drawn from a seed, so wavefronts drift apart as far as the kernel's own synchronisation
// lets them.
//
// Global -> LDS transfers (global_load_lds) complete asynchronously on the hardware, counted by vmcnt. Two extremes
// are modelled: EARLY, the bytes land when the instruction issues (exposes a transfer issued into a tile that
// another wavefront still reads), and LATE, they land only when the issuing lane executes the s_waitcnt that covers
// them (exposes a read that is not covered by a wait and a barrier). A kernel whose result is right under both, for
// several wavefront orders, has its tile ring, waits and barriers in the right places - which instructions it uses
// to get there is not what this checks (LDS reads return at once: registers reused under an outstanding read are the
// subject of tests/isa_hazards.py).
#pragma once
#include <stddef.h>
#include <stdint.h>
#include <math.h>
#include <string.h>
#include <algorithm>
#include <type_traits>

struct emu_dim3 { unsigned x, y, z; };

namespace emu {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kLanes = 64;

// ---- scheduler (emu.cpp)
const emu_dim3& thread_idx();
extern emu_dim3 g_block, g_grid;
extern int g_late_dma;             // 0 = EARLY, 1 = LATE
extern char* g_lds;                // the workgroup's LDS (160 KB)
void block_barrier();
void wave_barrier();
// all 64 lanes of the calling lane's wavefront deposit `bytes` bytes; returns the wavefront's table (64 x bytes),
// valid until the lane's next exchange
const void* wave_exchange(const void* mine, size_t bytes);
// asynchronous transfer bookkeeping
void dma_issue(const void* src, uint32_t lds_offset, int bytes);
void dma_wait(int allowed_outstanding);
typedef void (*kernel_fn)(void*);
// run `fn(arg)` on `threads` lanes for every block of a 1-D grid, with `lds` (160 KB) as the workgroup's LDS; returns 0,
// or 1 when the fibres deadlock
int run_grid(kernel_fn fn, void* arg, unsigned blocks, unsigned threads, unsigned seed, int late_dma, char* lds);

// ---- matrix instruction: D[i][j] = C[i][j] + sum_k A[i][k] B[k][j], 32 x 32 x 16. Lane l holds row l % 32 of A and
// column l % 32 of B for k = 8 (l / 32) .. + 7, and of C / D column l % 32, rows 8 (e / 4) + 4 (l / 32) + e % 4.
inline f16v mfma_32x32x16_f16(h8 a, h8 b, f16v c) {
    struct Ops { h8 a, b; } mine = {a, b};
    const Ops* all = static_cast<const Ops*>(wave_exchange(&mine, sizeof(mine)));
    const int lane = thread_idx().x & 63, col = lane & 31;
    f16v d = c;
    for (int e = 0; e < 16; ++e) {
        const int row = 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        float acc = 0.f;
        for (int k = 0; k < 16; ++k)
            acc += (float)all[row + 32 * (k / 8)].a[k % 8] * (float)all[col + 32 * (k / 8)].b[k % 8];
        d[e] = c[e] + acc;
    }
    return d;
}

// D = C + A B, 32 x 32 x 2 in fp32: lane l holds A[l % 32][l / 32] and B[l / 32][l % 32]; C / D as above.
inline f16v mfma_32x32x2_f32(float a, float b, f16v c) {
    struct Ops { float a, b; } mine = {a, b};
    const Ops* all = static_cast<const Ops*>(wave_exchange(&mine, sizeof(mine)));
    const int lane = thread_idx().x & 63, col = lane & 31;
    f16v d = c;
    for (int e = 0; e < 16; ++e) {
        const int row = 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        float acc = 0.f;
        for (int k = 0; k < 2; ++k) acc += all[row + 32 * k].a * all[col + 32 * k].b;
        d[e] = c[e] + acc;
    }
    return d;
}

inline int ds_bpermute(int byte_index, int value) {
    const int* all = static_cast<const int*>(wave_exchange(&value, sizeof(value)));
    return all[(byte_index >> 2) & 63];
}

inline unsigned long long ballot(bool p) {
    const int v = p;
    const int* all = static_cast<const int*>(wave_exchange(&v, sizeof(v)));
    unsigned long long m = 0;
    for (int i = 0; i < 64; ++i) m |= (unsigned long long)(all[i] != 0) << i;
    return m;
}

inline int readlane(int value, int lane) {
    const int* all = static_cast<const int*>(wave_exchange(&value, sizeof(value)));
    return all[lane];
}

inline float fdot2(_Float16 a0, _Float16 a1, _Float16 b0, _Float16 b1, float c) {
    return (float)a0 * (float)b0 + (float)a1 * (float)b1 + c;
}

}  // namespace emu

// ---- what the kernel sources see
#define __global__
#define __device__
#define __host__
#define __shared__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __restrict__
typedef emu_dim3 dim3;
#define threadIdx (emu::thread_idx())
#define blockIdx (emu::g_block)
#define gridDim (emu::g_grid)
#define __syncthreads() emu::block_barrier()
#define __builtin_amdgcn_s_barrier() emu::block_barrier()
#define __builtin_amdgcn_wave_barrier() emu::wave_barrier()
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) emu::mfma_32x32x16_f16(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) emu::mfma_32x32x2_f32(a, b, c)
#define __builtin_amdgcn_ds_bpermute(i, v) emu::ds_bpermute(i, v)
#define __builtin_amdgcn_ballot_w64(p) emu::ballot(p)
#define __builtin_amdgcn_readlane(v, l) emu::readlane(v, l)
#define __builtin_amdgcn_fdot2(a, b, c, clamp) emu::fdot2((a)[0], (a)[1], (b)[0], (b)[1], c)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_update_dpp(o, v, c, r, b, bc) (v)   /* wave reductions are not run here */
/* global -> LDS transfer of `size` bytes per lane: lane l's piece lands at the LDS pointer + size * l */
#define __builtin_amdgcn_global_load_lds(g, l, size, offset, aux) \
    emu::dma_issue((const void*)(g), (uint32_t)((const char*)(l) - emu::g_lds) + (size) * (threadIdx.x & 63), size)
inline unsigned long long wall_clock64() { return 0; }
inline uint32_t __umulhi(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
inline uint32_t __float_as_uint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
using std::max;
using std::min;

// host-side names the launch helpers in the kernel headers mention (never called here)
typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0, hipFuncAttributeMaxDynamicSharedMemorySize = 0, hipDeviceAttributeMultiprocessorCount = 0 };
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = 256; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, int, int) { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return ""; }
#define hipLaunchKernelGGL(...) ((void)0)
