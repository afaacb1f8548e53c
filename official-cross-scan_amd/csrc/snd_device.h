// Device-side helpers shared by the forward and backward kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "snd_scan.h"

namespace snd {

constexpr int kWave = 64;          // CDNA wavefront
constexpr int kRows = 8;           // rows per strip == row-checkpoint spacing
constexpr int kCkX = 8;            // column-checkpoint spacing == tile width
constexpr int kTile = kRows * kCkX;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Geometry of the opaque saved state (see snd_plan in snd_scan.h).
struct Geo {
    int nCX, nCY;                  // column tiles of kCkX, row strips of kRows
    int Hp, Wp;                    // padded inner extents nCY*kRows, nCX*kCkX
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

__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                            // round to nearest even
    return (uint16_t)(u >> 16);
}

// Typed element access.  The tile staging is the only code that touches caller tensors; everything
// after it is fp32.  Offsets inside one batch image are 32-bit (checked by the host entry points).
__device__ __forceinline__ float ldg(const float *base, int i) { return base[i]; }
__device__ __forceinline__ float ldg(const bf16_t *base, int i) { return bf16_to_f32(base[i].v); }
__device__ __forceinline__ float ldg(const f16_t *base, int i) { return (float)base[i]; }
__device__ __forceinline__ void stg(float *base, int i, float v) { base[i] = v; }
__device__ __forceinline__ void stg(bf16_t *base, int i, float v) { base[i].v = f32_to_bf16(v); }
__device__ __forceinline__ void stg(f16_t *base, int i, float v) { base[i] = (f16_t)v; }
// Same with the dtype chosen at run time (wave-uniform branch): used for out / dout, whose dtype
// may differ from the inputs' (fp32 or the input dtype).
__device__ __forceinline__ float ld_f32(const void *base, int i, int dt) {
    if (dt == SND_F32) return ((const float *)base)[i];
    if (dt == SND_BF16) return bf16_to_f32(((const uint16_t *)base)[i]);
    return (float)((const f16_t *)base)[i];
}
__device__ __forceinline__ void st_f32(void *base, int i, int dt, float v) {
    if (dt == SND_F32) ((float *)base)[i] = v;
    else if (dt == SND_BF16) ((uint16_t *)base)[i] = f32_to_bf16(v);
    else ((f16_t *)base)[i] = (f16_t)v;
}

// ---------------------------------------------------------------- math
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// softplus with the reference's threshold (fwd.cuh:223): log1p(e) = log(1+e) * e / ((1+e) - 1)
// keeps full relative accuracy for the tiny e = exp(x) that small time steps produce, using the
// hardware exp2/log2/rcp (about 1 ulp each).  Also returns the derivative sigmoid(x) (bwd.cuh:792).
__device__ __forceinline__ float softplus20(float x, float &dsp) {
    const float e = fast_exp2(x * kLog2e);
    const float w = 1.f + e;
    const float d = w - 1.f;
    const float rw = __builtin_amdgcn_rcpf(w);
    float sp = (d == 0.f) ? e : __builtin_amdgcn_logf(w) * kLn2 * (e * __builtin_amdgcn_rcpf(d));
    dsp = e * rw;
    if (x > 20.f) { sp = x; dsp = 1.f; }
    return sp;
}

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

// The same sum for four independent values at once, written out as fused v_add_f32_dpp steps.
// Interleaving the four values puts three instructions between a step and the next step of the
// same value, which covers the VALU-write -> DPP-read hazard; the leading s_nop covers the first.
#define SND_DPP4(ctrl)                                                   \
    "v_add_f32_dpp %0, %0, %0 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
    "v_add_f32_dpp %1, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
    "v_add_f32_dpp %2, %2, %2 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
    "v_add_f32_dpp %3, %3, %3 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
template <int NP> __device__ __forceinline__ void group_sum4(float &a, float &b, float &c, float &d) {
    if (NP == 16)
        asm("s_nop 1\n\t" SND_DPP4("quad_perm:[1,0,3,2]") SND_DPP4("quad_perm:[2,3,0,1]") SND_DPP4("row_half_mirror")
                SND_DPP4("row_mirror")
            : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    else if (NP == 8)
        asm("s_nop 1\n\t" SND_DPP4("quad_perm:[1,0,3,2]") SND_DPP4("quad_perm:[2,3,0,1]") SND_DPP4("row_half_mirror")
            : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    else { a = group_sum<NP>(a); b = group_sum<NP>(b); c = group_sum<NP>(c); d = group_sum<NP>(d); }
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

// Re-derive a thread's element maps from an opaque copy of its id.  Used at the top of each staging
// section so that the compiler recomputes a few integer ops per tile instead of hoisting dozens of
// loop-invariant addresses out of the tile loop and keeping (or spilling) them across it.
// Expects `tid`, `cbase`, `cend` in scope; defines wave, px, pr, pj, n, cl, cvalid, cc.
#define SND_THREAD_MAPS(NP)                                                        \
    int t_ = tid;                                                                  \
    asm volatile("" : "+v"(t_));                                                   \
    const int wave = t_ >> 6, px = t_ & 63, pr = px >> 3, pj = px & 7;             \
    const int n = t_ % (NP), cl = t_ / (NP);                                       \
    const int c_ = cbase + cl;                                                     \
    const bool cvalid = c_ < cend;                                                 \
    const int cc = cvalid ? c_ : cend - 1;                                         \
    (void)wave; (void)pr; (void)pj; (void)n; (void)cc

}  // namespace snd
