// Device-side helpers shared by the forward and backward kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "snd_scan.h"

namespace snd {

constexpr int kWave = 64;          // CDNA wavefront
constexpr int kRows = 8;           // storage rows per strip (row-checkpoint spacing is the tile extent, 8 or 7)
constexpr int kCkX = 8;            // storage columns per tile
constexpr int kTile = kRows * kCkX;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// The two kernel families lay the saved state out differently in tensors of the same shapes, so the forward leaves a
// tag in a word of x_sd that neither layout uses (its last one) and the backward compares it with its own: a
// backward of the other family would compute plausible-looking gradients from state it misreads; with the tag it
// multiplies dout by NaN instead, and every gradient - all are linear in dout - comes out NaN.
constexpr uint32_t kTagTile = 0x534E4431u, kTagWave = 0x534E4432u;
__host__ inline float *state_tag(float *x_sd, const snd_shape &sh) {
    if (x_sd == nullptr) return nullptr;
    snd_plan plan;
    return snd_make_plan(&sh, &plan) == SND_OK ? x_sd + plan.x_sd_elems - 1 : nullptr;
}
__device__ __forceinline__ float tag_poison(const float *tag, uint32_t mine) {
    return (tag == nullptr || *(const volatile uint32_t *)tag == mine) ? 1.f : __builtin_nanf("");
}

// Geometry of the opaque saved state (see snd_plan in snd_scan.h).  A plane is walked in tiles of
// te x te cells, te = 8 or 7: 7 where it leaves fewer padded cells (14, 28 and 7 are multiples of 7, not
// of 8: 23 % less work at those sizes).  Storage keeps 8 slots per tile row / column either way.
struct Geo {
    float *tag;                    // the family tag's place in the saved state (state_tag), or null
    int nCX, nCY;                  // column tiles, row strips (of te)
    int Hp, Wp;                    // inner extents of the saved state: nCY*8, nCX*8
    int te;                        // tile extent
    int nBands;                    // pipelined schedules: jobs per plane chunk (set by the launcher)
    int nQueues;                   // and the number of job queues: 8 (one per XCD) or 1
    int spinLimit;                 // polls a hand-over wait makes before it gives up (set by the launcher)
    int nSeg, segTiles;            // (backward, one strip per job) column segments per strip and tiles per segment
};
__host__ __device__ inline Geo make_geo(int H, int W) {
    const long long c8 = (long long)((H + 7) / 8) * ((W + 7) / 8) * 64, c7 = (long long)((H + 6) / 7) * ((W + 6) / 7) * 49;
    Geo g;
    g.te = c7 * 10 < c8 * 9 ? 7 : 8;   // a 7x7 tile costs a little more than 49/64 of an 8x8 one
    g.nCX = (W + g.te - 1) / g.te;
    g.nCY = (H + g.te - 1) / g.te;
    g.Hp = g.nCY * kRows;
    g.Wp = g.nCX * kCkX;
    g.nBands = 0;
    g.nQueues = 1;
    g.spinLimit = 1 << 21;
    g.nSeg = 1;
    g.segTiles = g.nCX;
    g.tag = nullptr;
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
// The same by byte offset from a block-uniform base pointer: base in scalar registers plus an
// unsigned 32-bit per-lane offset is one address mode of the vector memory instructions, so no
// 64-bit per-lane arithmetic is spent on addresses.  (The host entry points check that one batch
// image of every tensor spans fewer than 2^32 bytes and that row pitches fit 24-bit multiplies.)
__device__ __forceinline__ float ldg_b(const float *base, uint32_t off) { return *(const float *)((const char *)base + off); }
__device__ __forceinline__ float ldg_b(const bf16_t *base, uint32_t off) { return bf16_to_f32(((const bf16_t *)((const char *)base + off))->v); }
__device__ __forceinline__ float ldg_b(const f16_t *base, uint32_t off) { return (float)*(const f16_t *)((const char *)base + off); }
// The same load without the conversion, and the conversion: a value that is converted (or masked) where it is loaded
// is waited for there; kept raw, it is waited for where it is first needed.
__device__ __forceinline__ uint32_t ldraw_b(const float *base, uint32_t off) { return *(const uint32_t *)((const char *)base + off); }
__device__ __forceinline__ uint32_t ldraw_b(const bf16_t *base, uint32_t off) { return *(const uint16_t *)((const char *)base + off); }
__device__ __forceinline__ uint32_t ldraw_b(const f16_t *base, uint32_t off) { return *(const uint16_t *)((const char *)base + off); }
__device__ __forceinline__ float raw_to_f32(const float *, uint32_t r) { return __builtin_bit_cast(float, r); }
__device__ __forceinline__ float raw_to_f32(const bf16_t *, uint32_t r) { return __builtin_bit_cast(float, r << 16); }
__device__ __forceinline__ float raw_to_f32(const f16_t *, uint32_t r) { return (float)__builtin_bit_cast(f16_t, (uint16_t)r); }
// Four consecutive elements with one vector access (16 bytes of fp32, 8 bytes of 16-bit values), kept as raw bits
// until they are needed.  The address must be aligned to the access (the launchers check the tensors for it).
template <typename T> struct Raw4 { uint32_t w[sizeof(T)]; };           // 4 words, or 2 words of two 16-bit values each
__device__ __forceinline__ void ldraw4_b(Raw4<float> &q, const float *base, uint32_t off) {
    const uint4 v = *(const uint4 *)((const char *)base + off);
    q.w[0] = v.x; q.w[1] = v.y; q.w[2] = v.z; q.w[3] = v.w;
}
__device__ __forceinline__ void ldraw4_b(Raw4<bf16_t> &q, const bf16_t *base, uint32_t off) {
    const uint2 v = *(const uint2 *)((const char *)base + off);
    q.w[0] = v.x; q.w[1] = v.y;
}
__device__ __forceinline__ void ldraw4_b(Raw4<f16_t> &q, const f16_t *base, uint32_t off) {
    const uint2 v = *(const uint2 *)((const char *)base + off);
    q.w[0] = v.x; q.w[1] = v.y;
}
__device__ __forceinline__ void raw4_to_f32(const Raw4<float> &q, float (&o)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = __builtin_bit_cast(float, q.w[e]);
}
__device__ __forceinline__ void raw4_to_f32(const Raw4<bf16_t> &q, float (&o)[4]) {
    o[0] = __builtin_bit_cast(float, q.w[0] << 16); o[1] = __builtin_bit_cast(float, q.w[0] & 0xffff0000u);
    o[2] = __builtin_bit_cast(float, q.w[1] << 16); o[3] = __builtin_bit_cast(float, q.w[1] & 0xffff0000u);
}
__device__ __forceinline__ void raw4_to_f32(const Raw4<f16_t> &q, float (&o)[4]) {
    o[0] = (float)__builtin_bit_cast(f16_t, (uint16_t)q.w[0]); o[1] = (float)__builtin_bit_cast(f16_t, (uint16_t)(q.w[0] >> 16));
    o[2] = (float)__builtin_bit_cast(f16_t, (uint16_t)q.w[1]); o[3] = (float)__builtin_bit_cast(f16_t, (uint16_t)(q.w[1] >> 16));
}
__device__ __forceinline__ void stg4_b(float *base, uint32_t off, const float (&v)[4]) {
    *(float4 *)((char *)base + off) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void stg4_b(bf16_t *base, uint32_t off, const float (&v)[4]) {
    *(uint2 *)((char *)base + off) = make_uint2((uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16),
                                                (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16));
}
__device__ __forceinline__ void stg4_b(f16_t *base, uint32_t off, const float (&v)[4]) {
    const uint32_t a = __builtin_bit_cast(uint16_t, (f16_t)v[0]), b = __builtin_bit_cast(uint16_t, (f16_t)v[1]);
    const uint32_t c = __builtin_bit_cast(uint16_t, (f16_t)v[2]), d = __builtin_bit_cast(uint16_t, (f16_t)v[3]);
    *(uint2 *)((char *)base + off) = make_uint2(a | (b << 16), c | (d << 16));
}
__device__ __forceinline__ void stg_b(float *base, uint32_t off, float v) { *(float *)((char *)base + off) = v; }
__device__ __forceinline__ void stg_b(bf16_t *base, uint32_t off, float v) { ((bf16_t *)((char *)base + off))->v = f32_to_bf16(v); }
__device__ __forceinline__ void stg_b(f16_t *base, uint32_t off, float v) { *(f16_t *)((char *)base + off) = (f16_t)v; }
__device__ __forceinline__ float ld_f32_b(const void *base, uint32_t off, int dt) {
    const char *q = (const char *)base + off;
    if (dt == SND_F32) return *(const float *)q;
    if (dt == SND_BF16) return bf16_to_f32(*(const uint16_t *)q);
    return (float)*(const f16_t *)q;
}
__device__ __forceinline__ void st_f32_b(void *base, uint32_t off, int dt, float v) {
    char *q = (char *)base + off;
    if (dt == SND_F32) *(float *)q = v;
    else if (dt == SND_BF16) *(uint16_t *)q = f32_to_bf16(v);
    else *(f16_t *)q = (f16_t)v;
}
// A word of LDS that another wave of the block may have written since the last barrier: a plain LDS load.  (Read
// through a volatile generic pointer it becomes a flat load, and the wait for a flat load also covers every global
// load the wave has in flight.)
__device__ __forceinline__ int lds_peek(const int *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// float add to global memory, no value returned (one L2 atomic)
__device__ __forceinline__ void glb_add(float *p, float v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// a*b + c with 24-bit a, b (full-rate multiply-add; 32-bit integer multiplies are quarter rate)
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }

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

// Streaming 16-byte accesses for data that is written once and read once much later (saved state):
// marked non-temporal so that they do not displace the input lines that neighbouring tiles reuse.
typedef float v4f_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st4_stream(float *dst, float a, float b, float c, float d) {
    v4f_t v = {a, b, c, d};
    __builtin_nontemporal_store(v, (v4f_t *)dst);
}
__device__ __forceinline__ float4 ld4_stream(const float *src) {
    const v4f_t v = __builtin_nontemporal_load((const v4f_t *)src);
    return make_float4(v.x, v.y, v.z, v.w);
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
    else if (NP == 4)
        asm("s_nop 1\n\t" SND_DPP4("quad_perm:[1,0,3,2]") SND_DPP4("quad_perm:[2,3,0,1]")
            : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    else { a = group_sum<NP>(a); b = group_sum<NP>(b); c = group_sum<NP>(c); d = group_sum<NP>(d); }
}

// Reduce-scatter of eight values over an aligned group of 16 lanes (one DPP row): afterwards all
// four lanes of quad b (lanes 4b..4b+3 of the row) hold in v0, v1 the group totals of the original
// v[2b], v[2b+1]; v2..v7 are clobbered.  16 DPP adds instead of the 32 of eight broadcast sums:
//   lane bit 3: banks 0-1 fold their partner's v0..v3 in place, banks 2-3 write v4..v7 folded into v0..v3;
//   lane bit 2: banks 0,2 fold v0,v1 from the quad above, banks 1,3 write v2,v3 folded into v0,v1;
//   lane bits 1,0: plain butterfly on v0, v1.
// A DPP operand must not have been written by either of the two preceding VALU instructions; the
// instruction order below and the s_nops keep that distance.
#define SND_DPPA(d, s, ctrl, bank) "v_add_f32_dpp " d ", " s ", " s " " ctrl " row_mask:0xf bank_mask:" bank "\n\t"
__device__ __forceinline__ void group_scatter8(float &v0, float &v1, float &v2, float &v3, float &v4, float &v5,
                                               float &v6, float &v7) {
    asm("s_nop 1\n\t"
        SND_DPPA("%0", "%0", "row_ror:8", "0x3") SND_DPPA("%1", "%1", "row_ror:8", "0x3")
        SND_DPPA("%2", "%2", "row_ror:8", "0x3") SND_DPPA("%3", "%3", "row_ror:8", "0x3")
        SND_DPPA("%0", "%4", "row_ror:8", "0xc") SND_DPPA("%1", "%5", "row_ror:8", "0xc")
        SND_DPPA("%2", "%6", "row_ror:8", "0xc") SND_DPPA("%3", "%7", "row_ror:8", "0xc")
        SND_DPPA("%0", "%0", "row_shl:4", "0x5") SND_DPPA("%1", "%1", "row_shl:4", "0x5")
        SND_DPPA("%0", "%2", "row_shr:4", "0xa") SND_DPPA("%1", "%3", "row_shr:4", "0xa")
        "s_nop 0\n\t"
        SND_DPPA("%0", "%0", "quad_perm:[1,0,3,2]", "0xf") SND_DPPA("%1", "%1", "quad_perm:[1,0,3,2]", "0xf")
        "s_nop 0\n\t"
        SND_DPPA("%0", "%0", "quad_perm:[2,3,0,1]", "0xf") SND_DPPA("%1", "%1", "quad_perm:[2,3,0,1]", "0xf")
        : "+v"(v0), "+v"(v1), "+v"(v2), "+v"(v3), "+v"(v4), "+v"(v5), "+v"(v6), "+v"(v7));
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

// ---------------------------------------------------------------- strip pipeline
// With few (batch, channel) planes a plane is split into its row strips, one block per strip; the
// strips of a plane then run as a pipeline, each one tile behind the strip it depends on.
// Blocks take (plane chunk, strip) jobs from a ticket counter in dependency order, so the block a
// job waits for always holds an earlier ticket and is already running or finished.
// Sync words (int32, zeroed before the launch): [1] error flag, [4..11] ticket counters (one per job
// queue), [12 + plane chunk * strips + strip] count of tiles whose hand-over row the strip's block has
// written, and after those, in the same order, the count of column segments of the strip that are finished
// (backward with column-segmented strips, see strip_segments).
#ifndef SND_POLL_SLEEP
#define SND_POLL_SLEEP 16                           // s_sleep units (64 cycles) between polls
#endif
constexpr int kErrorWord = 1, kTicketWord = 4, kSyncHeader = 12;
constexpr int kSpinLimit = 1 << 21;                 // default polls (a memory round trip each) before giving up
// The limit launches use: kSpinLimit unless snd_debug_set_spin_limit() lowered it (tests of the time-out path).
int spin_limit();
// Timing studies of the tile kernels only (-DSND_TILE_ABLATE=<bits>, results wrong, never shipped): one memory
// stream of a kernel is switched off or pointed at one hot tile, and the time that goes away prices it.
// Forward: 1 no out stores, 2 staging loads from tile (0,0), 4 no checkpoint stores, 8 row-above loads from one
// tile.  Backward: 1 no dB/dC atomics, 2 staging loads from tile (0,0), 4 no du/ddelta stores, 8 checkpoint loads
// from one tile; (vector staging) 16 no loads of B and C, 32 none of delta, u and dout, 64 none of the halo of
// delta - their registers hold a constant instead.
#ifndef SND_TILE_ABLATE
#define SND_TILE_ABLATE 0
#endif
__host__ __device__ inline int64_t sync_words(int64_t nPlaneChunks, int nStrips) {
    // per (plane chunk, strip): tiles handed over, then column segments finished
#ifdef SND_PIPE_TRACE   // timing study only: 4 extra words per job (start, end, time spent waiting, -)
    return (kSyncHeader + 6 * nPlaneChunks * nStrips + 3) / 4 * 4;
#else
    return (kSyncHeader + 2 * nPlaneChunks * nStrips + 3) / 4 * 4;
#endif
}

// Data handed from one block to another inside a launch is written and read with agent-scope
// relaxed atomics (they go through to the coherence point and are never served from a stale line).
//
// Why no release / acquire fence is needed around the hand-over on gfx950:
//   * producer: the row is written with agent-scope atomic stores, which are performed at the agent's
//     coherence point and not held back in a wave-private or CU-private cache.  Every wave then executes
//     `s_waitcnt vmcnt(0)` (strip_stores_done): it does not pass this point before the coherence point has
//     acknowledged all of its stores.  The block barrier that follows makes that true for all waves of the
//     block, and only then does thread 0 move the count with an agent-scope atomic add.  So whoever can
//     observe the new count can observe the row: the count is issued after every store of the row has
//     completed, which is what a release fence would have waited for as well (it would in addition write
//     back the whole L2 working set of the block, which nothing here needs).
//   * consumer: the count is polled with agent-scope atomic loads, and the row is read with agent-scope
//     atomic loads (ld2_coherent) that are issued only after a poll has returned the expected value (the
//     loop exit is a branch on the loaded value, so the wave has waited for it).  Coherent loads are not
//     served from lines cached before the hand-over, which is what an acquire fence (a cache invalidate)
//     would have guaranteed for ordinary loads; no ordinary load ever touches the hand-over rows or counts.
//   * the compiler barrier at the end of strip_wait keeps the compiler from moving the row loads above the
//     poll; the hardware issues a wave's memory instructions in program order.
__device__ __forceinline__ void st2_coherent(float *dst, float a, float b) {
    const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, a) | ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
    __hip_atomic_store((uint64_t *)dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void ld2_coherent(const float *src, float &a, float &b) {
    const uint64_t v = __hip_atomic_load((const uint64_t *)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    a = __builtin_bit_cast(float, (uint32_t)v);
    b = __builtin_bit_cast(float, (uint32_t)(v >> 32));
}
__device__ __forceinline__ float ld1_coherent(const float *src) {
    return __builtin_bit_cast(float, __hip_atomic_load((const uint32_t *)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// Publish in two steps: every wave waits for its own hand-over stores to complete (vmcnt 0) before
// it reaches the block barrier; after the barrier one thread moves the count.
__device__ __forceinline__ void strip_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void strip_signal(int *count) {
    if (threadIdx.x == 0) __hip_atomic_fetch_add(count, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
#ifdef SND_PIPE_TRACE
#define SND_TRACE_ARG , int &trace_wait_
#define SND_TRACE_PASS , trace_wait_
#define g_wait_ticks trace_wait_
#else
#define SND_TRACE_ARG
#define SND_TRACE_PASS
#endif
// Wait until *count >= need.  `seen` caches the last value read (counts only grow), so a consumer
// that runs well behind its producer polls once per strip, not once per tile.  Bounded: after
// `limit` polls the error word (sync word kErrorWord) is set and the wave goes on so that the grid
// always drains; `dead` then disables further waits.  A block that gave up replaces every row it
// should have been handed by NaN (see the callers), so the outputs downstream of a timed-out wait are
// NaN and never plausible-looking numbers; the error word says why (snd_workspace_error reads it).
__device__ __forceinline__ void strip_wait(const int *count, int need, int &seen, int *sync, bool &dead, int limit SND_TRACE_ARG) {
    if (dead || seen >= need) return;
#ifdef SND_PIPE_TRACE
    const long long t0_ = wall_clock64();
#endif
    int polls = 0;
    while ((seen = __hip_atomic_load(count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) < need) {
        __builtin_amdgcn_s_sleep(SND_POLL_SLEEP);
        if (++polls > limit) {
            dead = true;
            __hip_atomic_store(sync + kErrorWord, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        }
    }
    asm volatile("" ::: "memory");
#ifdef SND_PIPE_TRACE
    g_wait_ticks += (int)(wall_clock64() - t0_);
#endif
}
// Take the next job.  Jobs are (plane chunk, band) in band-major order, so the job a block waits for
// always holds an earlier ticket of the same queue: it is running or finished.  With many (batch, group)
// pairs there is one queue per XCD (blocks are dealt round-robin to the XCDs, each with its own L2),
// holding the pairs congruent to it, so that all chunks and bands of a pair - they stream the same B/C
// planes - run on one XCD as in the whole-plane schedule; a block whose own queue is empty takes from
// the next one.  Returns false when no job is left (every block makes at most nQueues draws).
// With column segments (nSeg > 1; one strip per band, one queue) a job is (plane chunk, strip, segment) and the
// tickets run in the order of the earliest step a job can start at, strip + segment * segTiles (strips and segments
// counted in the order they are walked): both jobs a job waits for - the same segment of the strip before it and
// the segment before it of its own strip - have a smaller key, hence an earlier ticket.
__device__ __forceinline__ bool draw_job(int *sync, int nPairs, int nChunks, int nBands, int nQ, int &pair, int &chunk,
                                         int &band, int nSeg = 1, int segTiles = 0, int *seg = nullptr) {
    __shared__ int sJob[3];
    if (threadIdx.x == 0) {
        int q = blockIdx.x & (nQ - 1), t = -1;
        for (int k = 0; k < nQ; ++k) {
            const int jobs = ((nPairs - q + nQ - 1) / nQ) * nChunks * nBands * nSeg;
            if (jobs > 0) {
                const int got = __hip_atomic_fetch_add(sync + kTicketWord + q, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (got < jobs) { t = got; break; }
            }
            q = (q + 1) & (nQ - 1);
        }
        int sg = 0;
        if (nSeg > 1 && t >= 0) {                   // ticket -> (key, segment, plane chunk); the band follows from the key
            const int per = ((nPairs - q + nQ - 1) / nQ) * nChunks;
            int rem = t, key = 0;
            for (;; ++key) {
                int cnt = 0;
                for (int g = 0; g < nSeg; ++g) cnt += (key - g * segTiles >= 0 && key - g * segTiles < nBands);
                if (rem < cnt * per) break;
                rem -= cnt * per;
            }
            int gi = rem / per;
            rem -= gi * per;
            for (sg = 0; sg < nSeg; ++sg)
                if (key - sg * segTiles >= 0 && key - sg * segTiles < nBands && gi-- == 0) break;
            t = (key - sg * segTiles) * per + rem;  // the ticket this (band, plane chunk) has without segments
        }
        sJob[0] = t;
        sJob[1] = q;
        sJob[2] = sg;
    }
    __syncthreads();
    const int t = sJob[0], q = sJob[1];
    if (t < 0) return false;
    if (seg) *seg = sJob[2];
    const int per_band = ((nPairs - q + nQ - 1) / nQ) * nChunks;
    band = t / per_band;
    const int r = t - band * per_band;
    pair = (r / nChunks) * nQ + q;
    chunk = r - (r / nChunks) * nChunks;
    return true;
}
__host__ inline int job_queues(int nPairs) { return nPairs >= 16 ? 8 : 1; }
// Column segments per strip of the backward's strip pipeline (1 = whole strips).  A block that has drawn a strip
// holds its slot while it waits for the strip before it, so with more strip jobs than block slots the last strips of
// every plane start late (2 x 192 channels of 200 x 336: 600 strips of 42 tiles on 512 slots take 87 tile steps where
// the work is 49 and the chain of one plane 66).  Cut into segments of fewer tiles - the carried column state goes
// from one segment's block to the next through the workspace - the same jobs pack into 70 steps.  Decided by running
// the ticket order through a list-scheduling model (unit tile time, `slots` blocks at once; cached per shape):
// segments are taken where the model gains at least 8 %.  (256 channels of 512 x 512: 159 steps either way.)
int strip_segments(int64_t nPlaneChunks, int nStrips, int nTilesX, int64_t slots, int nQueues);
// floats of one strip's carried column state in the workspace (G, Gs, a of eight rows and the corner G per lane of a
// 256-thread block, as 8-byte words of all lanes one after the other)
constexpr int kColStateFloats = 13 * 2 * 256;
// Enqueue a fill kernel that zeroes n int32 words (defined with the C entry points).
int zero_words(int *p, int64_t n, hipStream_t stream);
// Per-device set-up (kernel attributes, the address of the static scratch array), done by snd_init() or
// by the first call that needs it on a device.  Returns an snd_status.
int ensure_device_ready();
// How a launch is scheduled (snd_fwd_params::schedule): one block per plane chunk walking all its
// strips, or one block per strip with the strips of a plane pipelined.
enum { kSchedAuto = 0, kSchedPlane = 1, kSchedStrips = 2, kSchedBands = 3 };
// Strip pipelining pays while whole-plane blocks leave the chip short of waves: always below 128 plane blocks, and
// up to 0.8 x the backward's block slots (410 of 512 for the 16-state kernels) when the strips of a plane give at
// least two blocks' worth of work side by side - a plane of nStrips x nTilesX tiles keeps
// nStrips*nTilesX / (nStrips + nTilesX - 1) of its strips busy on average (7x7 tiles: 3.8, 4x4: 2.3, 2x2: 1.3).
// Measured (16 states, fp32, 192 channels of 56x56, fwd + bwd ms, whole planes / strips): 192 plane blocks
// 0.93 / 0.61, 288: 1.19 / 0.83, 384: 1.24 / 1.08, 480: 1.31 / 1.35, 768: strips 1.07x slower; 384 blocks of 28x28:
// 0.36 / 0.31; 384 blocks of 14x14 (two strips): 0.097 / 0.116.  A strip waits for the strip above at every tile,
// which costs more than it gains once the planes alone fill the chip.
__host__ inline bool use_strip_pipeline(int schedule, int64_t planeBlocks, int nStrips, const void *sync, int nTilesX = 0,
                                        int64_t bwdSlots = 512) {
    if (schedule == kSchedPlane || sync == nullptr || nStrips < 2) return false;
    if (schedule == kSchedStrips) return true;
    if (planeBlocks < 128 || (planeBlocks < 256 && nStrips >= 16)) return true;
    const bool wide = nTilesX > 0 && (int64_t)nStrips * nTilesX >= 2 * ((int64_t)nStrips + nTilesX - 1);
    return wide && planeBlocks * 5 <= bwdSlots * 4;
}

// Jobs per plane chunk: 0 = one block walks the whole plane, nStrips = one strip per job, 2-4 = bands of
// strips.  A kernel holds `slots` blocks at once on the 256 CUs (backward 512; forward 768, or 1536 with
// the 128-thread blocks of the 8-state kernels).  With more plane chunks than slots the last round of
// whole-plane blocks leaves slots idle (backward, 768 chunks: two rounds, the second half empty);
// cutting every plane into a few bands of strips, handed over like strips but only at band ends, lets
// the ticket order pack them (768 x 2 bands: three rounds of half the length).
// Cost of q = jobs / slots rounds of equal jobs, in job lengths: full rounds cost one each; a last, partly filled
// round runs faster, because a block shares its CU with fewer others (k of the L blocks a CU holds: a share
// `serial` of a block's time does not depend on k - 0.6 in the issue-bound backward, where one block per CU takes
// 0.83 of the time it takes beside a second one, 0.15 in the bandwidth-bound forward); a round after the first
// costs a tenth more (tail of the round before).  Measured, 192 channels of 56x56, 16 states, whole planes, in
// units of a full round: backward 1.72 / 1.74 / 1.75 / 2.09 / 2.13 / 2.74 / 3.16 / 3.25 at 576 / 672 / 768 / 864 /
// 960 / 1152 / 1344 / 1536 plane chunks on 512 slots; forward 0.71 / 0.95 / 0.99 / 1.00 / 1.34 / 1.36 / 1.62 / 1.89 /
// 1.97 at 480 .. 1536 on 768 slots.
__host__ inline double rounds_cost(double q, int perCU, double serial) {
    const double full = (double)(int64_t)q, frac = q - full;
    if (frac < 1e-9) return full;
    int k = (int)(frac * perCU + 0.999999);
    if (k > perCU) k = perCU;
    return full + serial + (1.0 - serial) * k / perCU + (full >= 1.0 ? 0.1 : 0.0);
}
__host__ inline int band_count(int schedule, int64_t nPairs, int nChunks, int nStrips, const void *sync, int64_t slots,
                               int nTilesX = 0, int64_t bwdSlots = 512) {
    const int64_t planeBlocks = nPairs * nChunks;
    if (schedule == kSchedPlane || sync == nullptr || nStrips < 2) return 0;
    if (schedule == kSchedStrips) return nStrips;
    if (schedule != kSchedBands && use_strip_pipeline(kSchedAuto, planeBlocks, nStrips, sync, nTilesX, bwdSlots)) return nStrips;
    const bool forward = slots > bwdSlots;
    const int perCU = (int)(slots / 256);
    const double serial = forward ? 0.15 : 0.6;
    // the forward holds more blocks than the backward: between the backward's slots and 0.8 x its own, whole planes
    // put a third block on some CUs while the strips of a wide plane spread evenly (576 plane chunks: 0.48 -> 0.44 ms)
    const bool wide = nTilesX > 0 && (int64_t)nStrips * nTilesX >= 2 * ((int64_t)nStrips + nTilesX - 1);
    if (schedule != kSchedBands && forward && wide && planeBlocks > bwdSlots && planeBlocks * 5 <= slots * 4) return nStrips;
    // the 8-state forward (six 128-thread blocks per CU) prefers strips up to one full round of wide planes: 192 channels
    // of 56x56, bf16, whole planes / strips 0.407 / 0.380 ms at 768 plane chunks, 0.825 / 0.704 at 1536 (fp32 0.415 /
    // 0.414, 0.883 / 0.783); 28x28 at 1536: 0.232 / 0.222; beyond a round whole planes or bands are as good or better
    if (schedule != kSchedBands && forward && perCU >= 6 && wide && planeBlocks <= slots) return nStrips;
    // whole planes: every (batch, group) pair is pinned to one XCD (an eighth of the slots), so the rounds
    // are those of the fullest XCD (backward, 340 pairs x 3 chunks: 129 blocks there, three rounds)
    int best = 1;
    double best_cost = rounds_cost((double)((nPairs + 7) / 8 * nChunks) / (double)(slots / 8), perCU, serial);
    for (int nb = 2; nb <= 4 && nb <= nStrips; ++nb) {
        // rounds of jobs of length 1/nb (drawn from queues that balance the XCDs), never less than the
        // chain of one plane's bands, and a few percent per extra band for the hand-over
        double cost = rounds_cost((double)(planeBlocks * nb) / (double)slots, perCU, serial) / nb;
        cost = (cost < 1.0 ? 1.0 : cost) * (1.0 + 0.03 * (nb - 1));
        if (cost < best_cost * 0.96) { best = nb; best_cost = cost; }
    }
    if (schedule == kSchedBands) return best > 1 ? best : 2;
    return best > 1 ? best : 0;
}
// Blocks per CU by the state-lane count of the kernels (16, 8 or 4 lanes per channel): the backward is held
// to 2, 3, 4 by its LDS, the forward to 3, 6, 6.
__host__ inline int64_t bwd_slots(int dstate) { return dstate > 8 ? 512 : dstate > 4 ? 768 : 1024; }
__host__ inline int bwd_band_count(int schedule, int64_t nPairs, int nChunks, int nStrips, const void *sync, int dstate, int nTilesX = 0) {
    return band_count(schedule, nPairs, nChunks, nStrips, sync, bwd_slots(dstate), nTilesX, bwd_slots(dstate));
}
__host__ inline int fwd_band_count(int schedule, int64_t nPairs, int nChunks, int nStrips, const void *sync, int dstate, int nTilesX = 0) {
    return band_count(schedule, nPairs, nChunks, nStrips, sync, dstate > 8 ? 768 : 1536, nTilesX, bwd_slots(dstate));
}


// ---------------------------------------------------------------- row-segment wavefront (1-4 states per channel)
// With one to four states per channel a lane-per-(channel, state) mapping leaves most of the machine idle
// (256 channels x 1 state of a 512x512 plane are 256 lanes of work).  The second kernel family turns the
// plane itself into the parallel axis: the 64 lanes of a wave are 64 consecutive columns of one row (a
// row segment), the states of the channel live in registers of the lane, rows are taken one after the
// other, and the segments of a plane - one wave each, up to eight per block - advance as an anti-diagonal
// wavefront: wave w works on row i while wave w+1 works on row i-2 (forward; mirrored in the backward).
// Inside a segment the recurrence along the row, h_j = a_j*h_{j-1} + y_j, is resolved by a wave-wide
// inclusive scan of the affine maps (a_j, y_j) in six DPP steps (row_shr 1, 2, 4, 8, row_bcast 15, 31);
// neighbours in the row come from wave_shr:1 / wave_shl:1; the state at a segment's last column goes to
// the next wave through a few LDS words per row.
struct WaveGeo {
    float *tag;                    // the family tag's place in the saved state (state_tag), or null
    int nseg;                      // row segments a block of this launch works on (its waves per plane)
    int nsegAll;                   // row segments of a plane: ceil(W / (64 * cpl)); more than kMaxSeg: a wide plane, whose
                                   // segments are taken in column groups of at most kMaxSeg, one launch per group
    int seg0;                      // first segment of this launch's column group
    int extL, extR;                // whether a column group lies to the left / right of this launch's
    float *colh, *cols;            // (wide planes, forward) where column groups hand over h, a and s: the saved state
                                   // x, x_sd themselves, or a workspace of the same layout when no state is saved
    float *bcol;                   // (wide planes, backward) G, Gs, a at the first column of every column group;
                                   // (split planes, backward) the same as tagged words, see wave_bwd_split()
    int *sync;                     // (split planes) the workspace's sync words (error word) and the bound of a wait
    int spinLimit;
    int R;                         // rows per band (wave_band_rows): row-checkpoint spacing = rows the backward holds in registers
    int nBands;                    // ceil(H / R)
    int Hp, Wp;                    // nBands * R, nseg * 64 * cpl / planes per wave
    int cpl;                       // columns per lane: 1, or 2 (a lane owns two neighbouring columns: the scan and every
                                   // per-row overhead are paid once per two cells, and loads are twice as wide)
    int rg, rd, gshift, xcd;       // set by the launchers (wave_geo_channels): channels per group, channels per delta
                                   // channel, log2(groups) or -1, the block mapping (wave_job2) - divisions a wave
                                   // of a 7-row plane would spend a fifth of its instructions on
};
constexpr int kSeg = 64;
constexpr int kMaxSeg = 8;
constexpr int kOneWaves = 4;         // waves per block of the forward's one-segment instantiation
// Rows per band of the backward = spacing of the forward's row checkpoints.  The backward keeps a band's h, s, a and
// inputs of every state in registers, and what it gains from short bands is waves per SIMD: with one state 8 rows take
// 172-190 registers (two waves per SIMD), 4 rows 114-120 (four) - measured 13 to 39 % off the backward from 56x56 down
// to 7x7 planes, nothing at 512x512 x 256 channels (one block per CU either way), the forward within +-6 %; with two and
// four states 2 rows instead of 4 take 10 to 20 % off the backward.  The forward walks bands of its own height
// (load groups and wavefront steps) whatever the spacing and only stores the checkpoints more often: 4 rows with one
// and two states (2-row bands cost it 5 to 30 %), 2 rows with three and four, where the registers of a 4-row load
// group leave two waves per SIMD (192-245 registers; 64x192x56x56, four states: 0.352 -> 0.303 ms).
__host__ __device__ constexpr int wave_band_rows(int N) { return N <= 1 ? 4 : 2; }
__host__ __device__ constexpr int wave_fwd_rows(int N) { return N <= 2 ? 4 : 2; }
// Two columns per lane for one state and rows of 514 to 1024 columns (an even number): eight waves then still
// cover a row.  Narrower rows keep one column per lane - measured at 256 planes of 512 x 512: the same forward
// time and a 1.5 x slower backward with two, whose doubled per-lane state leaves one wave per SIMD.  Decided by
// the shape alone, because the saved state's segment boundaries follow from it.
// Rows wider still (wide planes) keep one column per lane: their segments are taken in column groups anyway.
__host__ __device__ inline int wave_cpl(int W, int N) { return (N <= 1 && W > kSeg * kMaxSeg && W <= 2 * kSeg * kMaxSeg && W % 2 == 0) ? 2 : 1; }
__host__ __device__ inline bool wave_family_fits(int W, int N) { return N <= 4; }
// A wide plane: more row segments than a block has waves.  Its segments are taken in column groups of kMaxSeg, left to
// right in the forward and right to left in the backward, one launch per group (the stream orders them); what crosses a
// group boundary - h, s, a of the column on its left (forward), G, Gs, a of the column on its right (backward), per row
// and state - goes through global memory instead of LDS.
__host__ __device__ inline bool wave_wide(int W, int N) { return (W + kSeg * wave_cpl(W, N) - 1) / (kSeg * wave_cpl(W, N)) > kMaxSeg; }
__host__ __device__ inline int wave_groups(int nsegAll) { return (nsegAll + kMaxSeg - 1) / kMaxSeg; }
// Planes per wave: narrow planes (one segment, at most 32 / 16 / 7 columns) are packed two / four / eight to a wave,
// plane q of a wave in lanes q*32.. / q*16.. / q*8.. (both kernels of a pair pack alike: the row checkpoints are as
// wide as a plane's lanes).  With eight planes the first lane of a plane is a barrier lane (wave_scan3_pk) and its
// columns are in lanes 1..7.
__host__ __device__ inline int wave_pack(const WaveGeo &g, int W) { return g.cpl == 1 && g.nsegAll == 1 ? (W <= 7 ? 8 : W <= 16 ? 4 : W <= 32 ? 2 : 1) : 1; }
__host__ __device__ inline WaveGeo make_wave_geo(int H, int W, int N) {
    WaveGeo g;
    g.cpl = wave_cpl(W, N);
    g.nsegAll = (W + kSeg * g.cpl - 1) / (kSeg * g.cpl);
    g.nseg = g.nsegAll < kMaxSeg ? g.nsegAll : kMaxSeg;
    g.seg0 = 0; g.extL = g.extR = 0;
    g.colh = g.cols = g.bcol = nullptr;
    g.sync = nullptr; g.spinLimit = 0;
    g.R = wave_band_rows(N);
    g.nBands = (H + g.R - 1) / g.R;
    g.Hp = g.nBands * g.R;
    g.Wp = g.nsegAll * kSeg * g.cpl / wave_pack(g, W);   // (packed planes: a row checkpoint is the plane's own lanes wide)
    g.rg = g.rd = 1; g.gshift = 0; g.xcd = 0;
    g.tag = nullptr;
    return g;
}
// Saved state of this family, per (batch, channel, state) plane, fp32 (S = 64 * cpl columns per segment):
//   x    [segment w][2][Hp]   h, then a, at column S*w-1 of every row (what segment w needs from its left)
//   x_sd [segment w][2][Hp]   s at the same places (second half unused)
//   x_v  [band][Wp]           h on the last row of every band (the backward recomputes a of that row from delta)
typedef float wave_f2 __attribute__((ext_vector_type(2)));
__host__ __device__ inline int64_t wave_x_plane(const WaveGeo &g) { return (int64_t)g.nsegAll * 2 * g.Hp; }
// (wide planes, backward) the hand-over between column groups, per (batch, channel, state) plane:
//   bcol [group q][3][Hp]   G, Gs, a at the first column of group q on every row (written by group q, read by group q-1)
__host__ __device__ inline int64_t wave_bcol_plane(const WaveGeo &g) { return (int64_t)wave_groups(g.nsegAll) * 3 * g.Hp; }
// Split planes (backward).  Few planes of eight segments with one or two states - 256 planes of 512 x 512 are
// one block of eight waves per CU - leave no room for two channels in a block, which is what halves the dB / dC
// atomics the kernel is bound by there.  Such a plane is cut in two halves of four segments: a block is two
// channels x one half, the two blocks of a channel pair run side by side in one launch, and the left half takes G, Gs,
// a of the right half's first column, band by band, through memory: 8-byte words {value, band + 1} that the right
// half's edge wave stores as it goes (no count, no wait for the stores) and an extra wave of the left half's block
// loads a band ahead and checks (all tags must be the band's; otherwise it loads again, a bounded number of times).
// The words are zeroed by a fill kernel before the launch.  Per (batch, channel, state) plane: [band][3][R] words.
__host__ __device__ inline bool wave_bwd_split(int batch, int dim, int W, int N) {
    const int cpl = wave_cpl(W, N), nseg = (W + kSeg * cpl - 1) / (kSeg * cpl);
    const int64_t planes = (int64_t)batch * dim;
    // (eight segments only: with six - two halves of three - the split measured 8-11 % slower than whole planes at
    // 1 x 192 x 300x384, two states, and 1 x 200 x 300x360; with eight 7-15 % faster, ragged widths included)
    // (at most 256 planes: with 512 planes of 512x512 - more blocks than run at once, so that left halves hold places
    // while they wait - the split took 0.79 ms against 0.71 for two channels in blocks of 16 waves)
    return cpl == 1 && N <= 2 && nseg == 8 && planes <= 256 && planes * nseg >= 1024;
}
__host__ __device__ inline int64_t wave_split_words(const WaveGeo &g) { return (int64_t)g.nBands * 3 * g.R * 2; }   // floats per plane
__host__ __device__ inline int64_t wave_xv_plane(const WaveGeo &g) { return (int64_t)g.nBands * g.Wp; }

// Block of the wavefront kernels -> (batch, group) pair and channel inside the group.  With many pairs all
// channels of a pair share an XCD (and its L2 copy of the pair's B / C planes) as in xcd_job; with few pairs
// that would leave XCDs idle, so the channels are dealt over all of them (B / C of few pairs are small).
__host__ inline int wave_grid(int nPairs, int rg) { return (nPairs >= 16 || (nPairs & 7) == 0) ? xcd_grid(nPairs, rg) : nPairs * rg; }
// The same mapping without a division: a grid of (8 * chunks, ceil(pairs / 8)) blocks is dispatched x first, so block
// (x, y) is the (8 * (y * chunks + x / 8) + x % 8)-th and lands on XCD x % 8 like block 8 * k + xcd of the flat grid.
// (WaveGeo.xcd says which of the two mappings the launcher chose.)
__host__ inline bool wave_grid_xcd(int nPairs) { return (nPairs >= 16 || (nPairs & 7) == 0) && (nPairs + 7) / 8 <= 65535; }
__host__ inline dim3 wave_grid2(int nPairs, int nChunks) {
    if (wave_grid_xcd(nPairs)) return dim3(8 * nChunks, (nPairs + 7) / 8);
    return dim3(nChunks, nPairs < 65535 ? nPairs : 65535, (nPairs + 65534) / 65535);
}
__device__ __forceinline__ bool wave_job2(const WaveGeo &g, int nPairs, int &pair, int &chunk) {
    if (g.xcd) {
        pair = blockIdx.y * 8 + (blockIdx.x & 7);
        chunk = blockIdx.x >> 3;
    } else {
        pair = blockIdx.z * 65535 + blockIdx.y;
        chunk = blockIdx.x;
    }
    return pair < nPairs;
}
__host__ inline void wave_geo_channels(WaveGeo &g, int batch, int dim, int n_groups, int delta_dim) {
    g.xcd = wave_grid_xcd(batch * n_groups) ? 1 : 0;
    g.rg = dim / n_groups;
    g.rd = dim / delta_dim;
    g.gshift = -1;
    for (int k = 0; k < 16; ++k)
        if (n_groups == 1 << k) g.gshift = k;
}
// (batch, group) of a pair
__device__ __forceinline__ void wave_pair_split(const WaveGeo &g, int pair, int G, int &b, int &grp) {
    b = g.gshift >= 0 ? pair >> g.gshift : pair / G;
    grp = pair - b * G;
}
// Row inputs of the wavefront kernels wait in registers as raw bits for a band of rows and are converted
// where they are used (a conversion at the load would put the wait for the load there).  They are loaded
// without any lane condition: a load whose result is only needed under a lane condition is sunk into that
// condition by the compiler - a branch with a full wait behind every load.
// A lane's CPL neighbouring elements come with one load when the tensor's alignment allows it (VEC: 4 bytes for
// two 16-bit values, 8 for two floats), else with one load per element.  Element e is the e-th in memory order.
template <typename T, int CPL, bool VEC> struct WaveRaw {
    static constexpr bool PACKED = CPL == 2 && VEC && sizeof(T) == 2;          // two 16-bit values in one register
    static constexpr int RW = PACKED ? 1 : CPL;
    // 16-bit values stay 16-bit until they are converted: widening them at the load would be an instruction per
    // value that has to wait for the load
    typedef typename std::conditional<sizeof(T) == 4 || PACKED, uint32_t, uint16_t>::type word_t;
    word_t w[RW];
};
template <typename T, int CPL, bool VEC>
__device__ __forceinline__ void wave_ld(WaveRaw<T, CPL, VEC> &q, const T *base, uint32_t off) {
    typedef WaveRaw<T, CPL, VEC> R;
    const char *a = (const char *)base + off;
    if (R::PACKED) {
        q.w[0] = *(const typename R::word_t *)a;
    } else if (CPL == 2 && VEC) {
        const uint2 v = *(const uint2 *)a;
        q.w[0] = v.x;
        q.w[R::RW - 1] = v.y;
    } else {
#pragma unroll
        for (int e = 0; e < CPL; ++e) q.w[e] = *(const typename R::word_t *)(a + e * sizeof(T));
    }
}
__device__ __forceinline__ float cvt_bits(const float *, uint32_t r) { return __builtin_bit_cast(float, r); }
__device__ __forceinline__ float cvt_bits(const bf16_t *, uint16_t r) { return __builtin_bit_cast(float, (uint32_t)r << 16); }
__device__ __forceinline__ float cvt_bits(const f16_t *, uint16_t r) { return (float)__builtin_bit_cast(f16_t, r); }
template <typename T, int CPL, bool VEC>
__device__ __forceinline__ float wave_elem(const WaveRaw<T, CPL, VEC> &q, int e) {
    typedef WaveRaw<T, CPL, VEC> R;
    const T *const tp = nullptr;
    if (R::PACKED) {
        const uint32_t v = q.w[0];
        if (std::is_same<T, bf16_t>::value) return __builtin_bit_cast(float, e == 0 ? v << 16 : v & 0xffff0000u);
        return cvt_bits(tp, (uint16_t)(e == 0 ? v : v >> 16));
    }
    return cvt_bits(tp, q.w[e < R::RW ? e : 0]);
}
// CPL values to consecutive elements in memory order
template <typename T, int CPL, bool VEC>
__device__ __forceinline__ void wave_st(T *base, uint32_t off, const float (&v)[CPL]) {
    char *a = (char *)base + off;
    if (CPL == 2 && VEC && sizeof(T) == 4) {
        *(float2 *)a = make_float2(v[0], v[CPL - 1]);
    } else if (CPL == 2 && VEC) {
        uint32_t lo, hi;
        if (std::is_same<T, bf16_t>::value) { lo = f32_to_bf16(v[0]); hi = f32_to_bf16(v[CPL - 1]); }
        else { lo = __builtin_bit_cast(uint16_t, (f16_t)v[0]); hi = __builtin_bit_cast(uint16_t, (f16_t)v[CPL - 1]); }
        *(uint32_t *)a = lo | (hi << 16);
    } else {
#pragma unroll
        for (int e = 0; e < CPL; ++e) stg_b(base, off + e * (uint32_t)sizeof(T), v[e]);
    }
}
// Stores and float atomics that take their own out-of-range lanes out: buffer instructions check a lane's offset against
// the descriptor's size in hardware and drop the lane if it is beyond, so a lane that is to do nothing is given the
// offset kBufOOB instead of a branch or an exec mask around the instruction.  The wave kernels' backward uses them for
// planes that are not whole bands x whole segments: with a branch around a store on some paths the waits the compiler
// derives for the prefetched loads have to assume the store was not issued (one counter, decremented in issue order),
// which cost such planes 12-38 % (64 x 192 x 56x63 against 56x64, one state; 2 x 256 x 512x250 against 512x256).
// The descriptor spans [base, base + kBufOOB); the scalar offset (a state's plane) is not part of the check.
constexpr uint32_t kBufOOB = 0xFFFFFFF0u;
typedef uint32_t buf_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buf_rsrc(void *base) { return __builtin_amdgcn_make_buffer_rsrc(base, 0, kBufOOB, 0x00020000); }
__device__ __forceinline__ void buf_add_f32(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t soff, float v) {
    __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, r, off, soff, 0);
}
__device__ __forceinline__ uint16_t bits16(const bf16_t *, float v) { return (uint16_t)f32_to_bf16(v); }
__device__ __forceinline__ uint16_t bits16(const f16_t *, float v) { return __builtin_bit_cast(uint16_t, (f16_t)v); }
__device__ __forceinline__ uint16_t bits16(const float *, float) { return 0; }
// CPL values to consecutive elements in memory order (wave_st through a buffer descriptor)
template <typename T, int CPL, bool VEC>
__device__ __forceinline__ void wave_st_buf(__amdgpu_buffer_rsrc_t r, uint32_t off, const float (&v)[CPL]) {
    const T *const tp = nullptr;
    if (CPL == 2 && VEC && sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b64((buf_u2){__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[CPL - 1])}, r, off, 0, 0);
    } else if (CPL == 2 && VEC) {
        __builtin_amdgcn_raw_buffer_store_b32((uint32_t)bits16(tp, v[0]) | ((uint32_t)bits16(tp, v[CPL - 1]) << 16), r, off, 0, 0);
    } else {
#pragma unroll
        for (int e = 0; e < CPL; ++e) {
            if (sizeof(T) == 4) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[e]), r, off + e * 4u, 0, 0);
            else __builtin_amdgcn_raw_buffer_store_b16(bits16(tp, v[e]), r, off + e * 2u, 0, 0);
        }
    }
}
// Block barrier for hand-overs through LDS only: waits for this wave's LDS traffic, not for its global loads
// and stores (the prefetched rows and the row just written stay in flight across it; __syncthreads would
// drain them at every step).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_old(float old, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
// v of the lane below (lane 0 keeps `edge`): the left neighbour when lanes run along the scan direction
__device__ __forceinline__ float from_prev_lane(float v, float edge) { return dpp_old<0x138, 0xF>(edge, v); }   // wave_shr:1
// v of the lane above (lane 63 keeps `edge`)
__device__ __forceinline__ float from_next_lane(float v, float edge) { return dpp_old<0x130, 0xF>(edge, v); }   // wave_shl:1

// Inclusive scan over the 64 lanes of the affine maps t -> a*t + y (and t -> a*t + s, sharing a):
// afterwards lane j holds a = prod_{k<=j} a_k, y = sum_{k<=j} (prod_{k<m<=j} a_m) y_k, s likewise, so that
// with a value c entering lane 0 from the left the recurrence's solution is a*c + y.
// Three interleaved chains per level keep two instructions between a VALU write and the DPP read of the
// same register (the hazard distance); lanes without a source (and rows masked off) keep their values.
#define SND_SCAN3_LVL(ctrl, rm)                                                  \
    "v_fmac_f32_dpp %0, %0, %2 " ctrl " row_mask:" rm " bank_mask:0xf\n\t"        \
    "v_fmac_f32_dpp %1, %1, %2 " ctrl " row_mask:" rm " bank_mask:0xf\n\t"        \
    "v_mul_f32_dpp %2, %2, %2 " ctrl " row_mask:" rm " bank_mask:0xf\n\t"
__device__ __forceinline__ void wave_scan3(float &y, float &s, float &a) {
    asm("s_nop 1\n\t" SND_SCAN3_LVL("row_shr:1", "0xf") SND_SCAN3_LVL("row_shr:2", "0xf") SND_SCAN3_LVL("row_shr:4", "0xf")
            SND_SCAN3_LVL("row_shr:8", "0xf") SND_SCAN3_LVL("row_bcast:15", "0xa") SND_SCAN3_LVL("row_bcast:31", "0xc")
        : "+v"(y), "+v"(s), "+v"(a));
}
// Packed planes: a wave holds PK = 2 or 4 planes of at most 32 or 16 columns, plane q in lanes q*64/PK ..; every
// plane is scanned on its own.  The levels that would cross into the next plane are left out: row_shr never leaves a
// 16-lane row, row_bcast:15 joins the two rows of a 32-lane plane.
template <int PK> __device__ __forceinline__ void wave_scan3_pk(float &y, float &s, float &a) {
    if (PK == 1) {
        wave_scan3(y, s, a);
    } else if (PK == 2) {
        asm("s_nop 1\n\t" SND_SCAN3_LVL("row_shr:1", "0xf") SND_SCAN3_LVL("row_shr:2", "0xf") SND_SCAN3_LVL("row_shr:4", "0xf")
                SND_SCAN3_LVL("row_shr:8", "0xf") SND_SCAN3_LVL("row_bcast:15", "0xa")
            : "+v"(y), "+v"(s), "+v"(a));
    } else if (PK == 4) {
        asm("s_nop 1\n\t" SND_SCAN3_LVL("row_shr:1", "0xf") SND_SCAN3_LVL("row_shr:2", "0xf") SND_SCAN3_LVL("row_shr:4", "0xf")
                SND_SCAN3_LVL("row_shr:8", "0xf")
            : "+v"(y), "+v"(s), "+v"(a));
    } else {
        // Eight planes of 8 lanes: row_shr carries lane 7 of a 16-lane row into lane 8, the first lane of the next
        // plane.  That lane is a barrier: it holds the map (a, y, s) = (0, 0, 0), which stays what it is under every
        // composition, and a lane whose range has reached it holds a = 0 and takes nothing from beyond it.  (Switching
        // lanes off in EXEC instead does not work: a DPP read of a disabled lane is an invalid source.)
        asm("s_nop 1\n\t" SND_SCAN3_LVL("row_shr:1", "0xf") SND_SCAN3_LVL("row_shr:2", "0xf") SND_SCAN3_LVL("row_shr:4", "0xf")
            : "+v"(y), "+v"(s), "+v"(a));
    }
}
// v of the lane below inside the lane's plane; the plane's first lane (`first`) keeps `edge`.
template <int PK> __device__ __forceinline__ float from_prev_lane_pk(float v, float edge, bool first) {
    if (PK == 1) return from_prev_lane(v, edge);
    // (eight planes: a plane's first lane is its barrier lane, whose own results are never used)
    if (PK == 4 || PK == 8) return dpp_old<0x111, 0xF>(edge, v);       // row_shr:1
    const float t = from_prev_lane(v, edge);
    return first ? edge : t;
}
// v of the lane above inside the lane's plane; the plane's last lane (`last`) keeps `edge`.
template <int PK> __device__ __forceinline__ float from_next_lane_pk(float v, float edge, bool last) {
    if (PK == 1) return from_next_lane(v, edge);
    // (eight planes: the lane after a plane's last is the next plane's barrier lane, which holds the zero edge)
    if (PK == 4 || PK == 8) return dpp_old<0x101, 0xF>(edge, v);       // row_shl:1
    const float t = from_next_lane(v, edge);
    return last ? edge : t;
}

// One row of a segment: t_j = a_j*t_{j-1} + y_j and the same with s_j, over the CPL columns of each of the 64
// lanes, lanes ascending in the direction of the recurrence, cy / cs entering the first column of lane 0.
// The CPL maps of a lane are composed first, one scan runs over the lanes, and the lane's columns are filled
// in from the value entering the lane.  Returns the solutions per column (the lane's last: oy[CPL-1]).
template <int CPL, int PK = 1>
__device__ __forceinline__ void wave_row_solve(const float (&a)[CPL], const float (&y)[CPL], const float (&sv)[CPL], float cy,
                                               float cs, float (&oy)[CPL], float (&os)[CPL]) {
    static_assert(PK == 1 || CPL == 1, "packed planes: one column per lane");
    float Y = y[0], S = sv[0], Ap = a[0];
#pragma unroll
    for (int k = 1; k < CPL; ++k) {
        Y = fmaf(a[k], Y, y[k]);
        S = fmaf(a[k], S, sv[k]);
        Ap *= a[k];
    }
    wave_scan3_pk<PK>(Y, S, Ap);
    const float ey = fmaf(Ap, cy, Y), es = fmaf(Ap, cs, S);      // at the lane's last column
    if (CPL > 1) {
        float ty = from_prev_lane(ey, cy), ts = from_prev_lane(es, cs);   // entering the lane
#pragma unroll
        for (int k = 0; k < CPL - 1; ++k) {
            ty = fmaf(a[k], ty, y[k]);
            ts = fmaf(a[k], ts, sv[k]);
            oy[k] = ty;
            os[k] = ts;
        }
    }
    oy[CPL - 1] = ey;
    os[CPL - 1] = es;
}

// Sum over the 64 / PK lanes of each packed plane; the total ends in the plane's last lane.
template <int PK> __device__ __forceinline__ float wave_sum_to_plane_last(float v) {
    if (PK == 8) {                                   // butterflies inside the 8 lanes: every lane ends with the total
        v += dpp_old<0xB1, 0xF>(0.f, v);             // quad_perm:[1,0,3,2]
        v += dpp_old<0x4E, 0xF>(0.f, v);             // quad_perm:[2,3,0,1]
        v += dpp_old<0x141, 0xF>(0.f, v);            // row_half_mirror
        return v;
    }
    v += dpp_old<0x111, 0xF>(0.f, v);
    v += dpp_old<0x112, 0xF>(0.f, v);
    v += dpp_old<0x114, 0xF>(0.f, v);
    v += dpp_old<0x118, 0xF>(0.f, v);
    if (PK <= 2) v += dpp_old<0x142, 0xA>(0.f, v);
    if (PK == 1) v += dpp_old<0x143, 0xC>(0.f, v);
    return v;
}
// Sum over the 64 lanes; the total ends in lane 63.
__device__ __forceinline__ float wave_sum_to_last(float v) {
    v += dpp_old<0x111, 0xF>(0.f, v);
    v += dpp_old<0x112, 0xF>(0.f, v);
    v += dpp_old<0x114, 0xF>(0.f, v);
    v += dpp_old<0x118, 0xF>(0.f, v);
    v += dpp_old<0x142, 0xA>(0.f, v);
    v += dpp_old<0x143, 0xC>(0.f, v);
    return v;
}

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
