// Device-side helpers shared by the forward and backward kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "snd_scan.h"

namespace snd {

constexpr int kWave = 64;          // CDNA wavefront
constexpr int kRows = 8;           // rows per strip == row-checkpoint spacing
constexpr int kCkX = 8;            // column-checkpoint spacing == backward tile width
constexpr float kLog2e = 1.4426950408889634f;

// Geometry of the opaque saved state (see snd_plan in snd_scan.h).
struct Geo {
    int nCX, nCY;                  // column tiles of kCkX, row strips of kRows
    int Hp, Wp;                    // padded inner extents: nCY*kRows, round_up(W, 4) (+4 slack)
};
__host__ __device__ inline Geo make_geo(int H, int W) {
    Geo g;
    g.nCX = (W + kCkX - 1) / kCkX;
    g.nCY = (H + kRows - 1) / kRows;
    g.Hp = g.nCY * kRows;
    g.Wp = g.nCX * kCkX;
    return g;
}

// ---------------------------------------------------------------- element types
struct bf16_t { uint16_t v; };
typedef _Float16 f16_t;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(f16_t x) { return (float)x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __builtin_bit_cast(float, (uint32_t)x.v << 16); }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float x) { return (f16_t)x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.v = (uint16_t)((u >> 16) | 0x40u); return r; }   // NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                                         // RNE
    r.v = (uint16_t)(u >> 16);
    return r;
}

// ---------------------------------------------------------------- math
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// softplus with the reference's threshold (fwd.cuh:223); log1pf keeps relative accuracy for
// the small deltas (1e-3) the operator is used with.
__device__ __forceinline__ float softplus20(float x) { return x <= 20.f ? log1pf(__expf(x)) : x; }

// ---------------------------------------------------------------- cross-lane sums (DPP)
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// Sum over aligned groups of NP consecutive lanes (NP a power of two <= 16); every lane of the
// group receives the total.  quad_perm[1,0,3,2], quad_perm[2,3,0,1], row_half_mirror, row_mirror.
template <int NP> __device__ __forceinline__ float group_sum(float v) {
    if (NP >= 2) v += dpp_mov<0xB1>(v);
    if (NP >= 4) v += dpp_mov<0x4E>(v);
    if (NP >= 8) v += dpp_mov<0x141>(v);
    if (NP >= 16) v += dpp_mov<0x140>(v);
    return v;
}

// Blocks are dealt round-robin to the 8 XCDs (each with its own L2).  Keep every chunk of one
// (batch, group) pair - they all stream the same B/C planes - on one XCD.
__device__ __forceinline__ bool xcd_job(int bid, int nPairs, int nChunks, int &pair, int &chunk) {
    const int xcd = bid & 7, k = bid >> 3;
    pair = (k / nChunks) * 8 + xcd;
    chunk = k % nChunks;
    return pair < nPairs;
}
__host__ inline int xcd_grid(int nPairs, int nChunks) { return ((nPairs + 7) / 8) * 8 * nChunks; }

}  // namespace snd
