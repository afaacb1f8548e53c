// Backward kernel of the 2D-CrossScan selective scan for gfx950.
//
// Computes the gradients the reference's selective_scan_bwd_kernel produces
// (kernels/selective_nd_scan/include/cusoflex/selective_scan_bwd_kernel_oflex.cuh:91-902).
// With G = a*g, Gs = a*gs and every out-of-range term zero, per (batch, channel, state) plane:
//     g[i,j]  = dout*C + G[i,j+1] + G[i+1,j] - 0.5*(a[i,j+1] + a[i+1,j])*G[i+1,j+1]      (:463-469,486-488)
//     gs[i,j] = -dout*C + Gs[i,j+1]                                                      (:710,722-724)
//     dbu     = g + gs + 0.25*dout*C                                                     (:513,749-754)
//     da*a    = g*(h - bu) + gs*(s - bu) - 0.5*a*(G[i+1,j]*h[i,j-1] + G[i,j+1]*h[i-1,j]) (:515-587,751-753)
//     ddelta  = sum_n (A*da*a + dbu*B*u), then * sigmoid(raw) under softplus             (:516,752,785-806)
//     du      = D*dout + delta' * sum_n dbu*B                                            (:211,514,750)
//     dB      = sum_{c in group} dbu*delta'*u        dC = sum_{c in group} dout*(h - s + 0.25*bu)   (:589-590,754-755)
//     dA      = sum_{b,i,j} delta'*da*a              dD = sum dout*u     ddelta_bias = sum ddelta    (:518,753,212,808-819)
// (g*(h-bu) is the reference's dx*a with a = (h-bu); the two -0.5 terms are the places a[i,j]
// enters its right and lower neighbours, which the reference scatters to ddelta_vals[nrow-1][i],
// ddelta_vals[nrow][i-1] and stitches across chunk seams; here they are gathered at the cell.)
//
// Organisation (not a translation): the same lane = one (channel, state) plane, TE x TE tile walk
// as the forward (TE = 8 or 7), in reverse.  For each tile a lane recomputes h from the forward's checkpoints (row above
// from x_v, column to the left from x, s from x_sd), one half of the tile (4 columns, then the rest) at a time into 32
// registers, and sweeps that half bottom-right to top-left.  The adjoint row handed to the strip
// above goes through a private global scratch row; the column handed to the tile on the left stays
// in registers.  dB/dC are reduced over a wave's channels with lane swaps, over the block's waves
// through LDS, and leave the block once per tile; du/ddelta are reduced over states by DPP and
// finished once per pixel by the thread that staged it.
// As in the forward, tiles are computed in full on zero-padded staging (dout = B = C = 0 outside
// the plane makes every adjoint there exactly zero), so the inner loops have no bounds checks.
#pragma once
#include <initializer_list>
#include <type_traits>
#include "snd_device.h"

namespace snd {

// Sum two sets of four values over the four 16-lane rows of a wave (its four channels when a row
// holds the 16 states of one channel): a reduce-scatter, row q of the wave ends with the totals of
// b[q] (in b0) and c[q] (in c0).  v_permlane32_swap exchanges the upper 32 lanes of its first
// operand with the lower 32 lanes of its second, v_permlane16_swap the odd 16-lane rows of the first
// with the even rows of the second; after either, first + second is the pair-sum of the value the
// lane keeps.  A swap must not read a register written by the two preceding VALU instructions and
// its results must not be read by the two following ones: the order and the s_nops keep that distance.
__device__ __forceinline__ void rows_scatter4x2(float &b0, float &b1, float &b2, float &b3, float &c0, float &c1,
                                                float &c2, float &c3) {
    asm volatile("s_nop 1\n\t"
                 "v_permlane32_swap_b32 %0, %2\n\t"
                 "v_permlane32_swap_b32 %1, %3\n\t"
                 "v_permlane32_swap_b32 %4, %6\n\t"
                 "v_permlane32_swap_b32 %5, %7\n\t"
                 "v_add_f32 %0, %0, %2\n\t"
                 "v_add_f32 %1, %1, %3\n\t"
                 "v_add_f32 %4, %4, %6\n\t"
                 "v_add_f32 %5, %5, %7\n\t"
                 "s_nop 0\n\t"
                 "v_permlane16_swap_b32 %0, %1\n\t"
                 "v_permlane16_swap_b32 %4, %5\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32 %0, %0, %1\n\t"
                 "v_add_f32 %4, %4, %5\n\t"
                 : "+v"(b0), "+v"(b1), "+v"(b2), "+v"(b3), "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3));
}
#ifndef SND_BWD_WAVES
#define SND_BWD_WAVES 2
#endif
#ifndef SND_KA8
#define SND_KA8 3
#endif
// VEC: the tile's inputs are staged, and du / ddelta stored, four columns at a time with one 16-byte (fp32) or
// 8-byte (16-bit) access per thread and tensor instead of one access per element - a quarter of the memory
// instructions and of their address arithmetic.  Needs 8x8 tiles, a width that is a multiple of four and tensors
// whose rows start on such boundaries (bwd_vec_ok); everything else takes the element-wise staging.
// SEG: (pipelined strips only) a job is a column segment of a strip; the carried column state goes from one
// segment's block to the next through the workspace (strip_segments).  A variant of its own, because the few
// registers it takes are registers the other variants do not have.
template <typename T, int NP, bool PIPE, int TE, bool VEC, bool SEG = false>
__global__ __launch_bounds__(16 * NP) __attribute__((amdgpu_waves_per_eu(SND_BWD_WAVES, SND_BWD_WAVES))) void bwd_kernel(const snd_bwd_params p, const Geo geo) {
    static_assert(!VEC || TE == 8, "vector staging needs 8x8 tiles");
    static_assert(!SEG || PIPE, "column segments belong to the strip pipeline");
    constexpr int WPB = NP / 4;                     // waves per block
    constexpr int CB = 16;                          // channels per block
    constexpr int NSTR = kTile + 4;
    // Pitches in floats, chosen for the 32 four-byte banks of LDS (a pitch of 64 would put every channel of a
    // wave in the same bank).  PCH: pixel arrays that the sweep reads as one float4 per channel (all lanes of a
    // channel the same address), so the channels of a wave must start 4 banks apart.  PCS: pixel arrays that
    // only the staging and the per-pixel epilogue touch, lane n of a channel at element n, so a channel takes NP
    // consecutive banks.  NSD: the dB/dC partial sums, which the 16-lane row q of a wave writes at element q of
    // a state's tile row, so states must start 2 (16 states) or 4 banks apart.
    constexpr int PCH = kTile + (NP == 16 ? 8 : 4);
    constexpr int PCS = kTile + NP;
    constexpr int NSD = NP == 16 ? kTile + 2 : kTile + 4;
    constexpr int NBC = 4;
    constexpr int NPX = kTile / NP;
    // delta' on the tile plus a one-cell halo: rows -1..8 at a pitch of 12 floats, column j at element DLO + j, so
    // that columns 0-3 and 4-7 of a row are each one aligned 16-byte read (channels of a wave 24 banks apart)
    constexpr int HG = 12, DLO = 4, DLP = 10 * HG;
    constexpr int NHALO = 4 * TE + 4, NHK = (NHALO + NP - 1) / NP;   // ring around the TE x TE tile
    constexpr int NCH = VEC ? kTile / 4 / NP : 0;   // (VEC) four-column chunks of a channel's tile per thread
    constexpr int NHV = (24 + NP - 1) / NP;         // (VEC) halo cells per thread: row above, row below, column to the left

    // A wave's channels (four with 16 states per channel, eight with 8) are reduced in registers and
    // every wave owns a partial dB/dC tile, written with plain stores.
    constexpr int NPART = WPB;
    extern __shared__ __align__(16) float smem[];
    float *sB = smem;                               // [NP][NSTR]
    float *sC = sB + NP * NSTR;
    float *sdB = sC + NP * NSTR;                    // [NPART][NP][NSD]
    float *sdC = sdB + NPART * NP * NSD;
    float *sDl = sdC + NPART * NP * NSD;            // [CB][DLP]
    float *sDu = sDl + CB * DLP;                    // [CB][PCH] delta' * u
    float *sU = sDu + CB * PCH;                     // [CB][PCS]
    float *sDo = sU + CB * PCS;                     // dout
    float *sSg = sDo + CB * PCH;                    // [CB][PCS] d softplus / d raw
    float *sQ = sSg + CB * PCS;                     // sum_n dbu*B
    float *sP = sQ + CB * PCH + 4;                  // sum_n A*da*a (4 banks off sQ: a wave writes both in one instruction)
    float *sRed = sP + CB * PCH;                    // [WPB]

    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = Dm / G, rd = Dm / sh.delta_dim;
    const int nChunks = (rg + CB - 1) / CB;
    int pair, chunk;
    int I_hi = geo.nCY - 1, I_lo = 0;               // strips this block walks, bottom to top
    int J_hi = geo.nCX - 1, J_lo = 0, seg = 0;      // and the tiles of a strip, right to left (a column segment of a pipelined strip)
    int *sync = (int *)p.workspace, *progress = nullptr, *segdone = nullptr;
    float *colstate = nullptr;
    const int64_t nSync = sync_words((int64_t)sh.batch * G * nChunks, geo.nCY);
    bool dead = false;
    int seen = 0;                                   // last progress count read (strip pipeline)
#ifdef SND_PIPE_TRACE
    int *trace_ = nullptr, trace_wait_ = 0;
#endif
    __shared__ int sSeen;                           // (pipelined) progress count of the strip below, as last polled
    __shared__ int sDead;                           // (pipelined) a hand-over wait of this block has timed out
    if (PIPE) {
        if (threadIdx.x == 0) { sSeen = 0; sDead = 0; }   // ordered before their readers by the barrier in draw_job
        // A job is a band of consecutive strips (one strip each in the fully pipelined case), drawn
        // bottom band first; band k from the bottom covers strips ceil(k*nCY/nBands) ..
        // ceil((k+1)*nCY/nBands)-1, counted from the bottom.
        int band;
        if (!draw_job(sync, sh.batch * G, nChunks, geo.nBands, geo.nQueues, pair, chunk, band, SEG ? geo.nSeg : 1, geo.segTiles, &seg)) return;
        const int nPC = sh.batch * G * nChunks;
        const int pc = pair * nChunks + chunk;
        I_hi = geo.nCY - 1 - (band * geo.nCY + geo.nBands - 1) / geo.nBands;
        I_lo = geo.nCY - ((band + 1) * geo.nCY + geo.nBands - 1) / geo.nBands;
        progress = sync + kSyncHeader + pc * geo.nCY;
        // (column-segmented strips: one strip per job) the segment's tiles, right to left; the carried column state
        // of the strip goes from segment to segment through one slot of the workspace
        if (SEG) {
            J_hi = geo.nCX - 1 - seg * geo.segTiles;
            J_lo = seg == geo.nSeg - 1 ? 0 : J_hi - geo.segTiles + 1;
            segdone = progress + nPC * geo.nCY;
            colstate = (float *)p.workspace + nSync + (int64_t)sh.batch * Dm * N * geo.Wp + ((int64_t)pc * geo.nCY + I_hi) * kColStateFloats;
        }
#ifdef SND_PIPE_TRACE
        trace_ = sync + kSyncHeader + 2 * nPC * geo.nCY + 4 * (pc * geo.nCY + I_hi);
        if (threadIdx.x == 0) trace_[0] = (int)wall_clock64();
#endif
    } else if (!xcd_job(blockIdx.x, sh.batch * G, nChunks, pair, chunk)) return;
    const int b = pair / G, g = pair - b * G;
    const int cbase = g * rg + chunk * CB, cend = (g + 1) * rg;
    // scan origin of this group (as in the forward): memory row = mrow(i) = r0m + rs*i, column = mcol(j)
    const bool fv = f.directions == SND_DIR_CORNERS && (g & 2), fh = f.directions == SND_DIR_CORNERS && (g & 1);
    const int r0m = fv ? H - 1 : 0, rs = fv ? -1 : 1, c0m = fh ? W - 1 : 0, cs = fh ? -1 : 1;
    auto mrow = [&](int r) { return mad24(r, rs, r0m); };
    auto mcol = [&](int c_) { return mad24(c_, cs, c0m); };

    const int tid = threadIdx.x, wave = tid >> 6;
    const int n = tid % NP, cl = tid / NP;
    const int c = cbase + cl;
    const bool cvalid = c < cend;
    const bool lvalid = cvalid && n < N;
    const int cc = cvalid ? c : cend - 1, nn = n < N ? n : N - 1;
    const int px = tid & 63, pr = px >> 3, pj = px & 7;

    const float Av = lvalid ? f.A[(int64_t)cc * f.A_d_stride + (int64_t)nn * f.A_dstate_stride] : 0.f;
    const float A2 = Av * kLog2e;
    const float ld = f.A_decay ? __log2f(f.A_decay[0]) : 0.f;
    const float Dv = f.D ? f.D[cc] : 0.f;
    const float bias = f.delta_bias ? f.delta_bias[cc / rd] : 0.f;
    const bool softplus = f.delta_softplus != 0;

    // per-batch-image base pointers (uniform) and 32-bit offsets inside the image
    const T *Bb = (const T *)f.B + (int64_t)b * f.B_batch_stride + (int64_t)g * f.B_group_stride;
    const T *Cb = (const T *)f.C + (int64_t)b * f.C_batch_stride + (int64_t)g * f.C_group_stride;
    const T *ub = (const T *)f.u + (int64_t)b * f.u_batch_stride;
    const T *db = (const T *)f.delta + (int64_t)b * f.delta_batch_stride;
    const int sh_do = p.dout_dtype == SND_F32 ? 2 : 1, esz_do = 1 << sh_do;
    const void *dob = (const char *)p.dout + (int64_t)b * p.dout_batch_stride * esz_do;
    T *dub = (T *)p.du + (int64_t)b * Dm * H * W;                    // du, ddelta: dense [b, c, H, W]
    T *ddb = (T *)p.ddelta + (int64_t)b * Dm * H * W;
    float *dBg = p.dB + ((int64_t)b * G + g) * N * H * W;            // dense [b, g, N, H, W]
    float *dCg = p.dC + ((int64_t)b * G + g) * N * H * W;
    // byte offsets inside the batch image: per-lane channel offsets (kept across the tile loop) and
    // row pitches / state strides in bytes
    constexpr int ESZ = (int)sizeof(T);
    const uint32_t cUb = (uint32_t)(f.u_shared ? cc - g * rg : cc) * (uint32_t)f.u_d_stride * ESZ, cDb = (uint32_t)(cc / rd) * (uint32_t)f.delta_d_stride * ESZ;
    // fused CrossMerge: dout is the gradient of the merged output (one channel per feature, shared by the groups);
    // the channel's weight is applied where dout is staged, and every gradient, being linear in dout, follows
    const bool merge = f.merge != 0;
    // (times NaN if the saved state was written by the other kernel family: see kTagTile)
    const float wm = (merge && f.merge_weights ? f.merge_weights[cc] : 1.f) * tag_poison(geo.tag, kTagTile);
    const uint32_t cDob = ((uint32_t)(merge ? cc - g * rg : cc) * (uint32_t)p.dout_d_stride) << sh_do;
    const uint32_t cGb = (uint32_t)cc * (uint32_t)(H * W) * ESZ;      // du, ddelta
    const int BhB = (int)f.B_h_stride * ESZ, ChB = (int)f.C_h_stride * ESZ, UhB = (int)f.u_h_stride * ESZ, DhB = (int)f.delta_h_stride * ESZ;
    const int DohB = (int)p.dout_h_stride << sh_do, WB = W * ESZ, W4 = W * 4;
    const int64_t BsB = f.B_dstate_stride * ESZ, CsB = f.C_dstate_stride * ESZ;
    const int64_t HW4 = (int64_t)H * W * 4;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);   // the wave index as a scalar

    // saved state and scratch, tile-major; inside a tile the lanes' values 0-3, then the lanes' values
    // 4-7 (as the forward writes: a wave's 16-byte accesses cover whole lines):
    //   x_v [b][I][J][half][c][n][4 cols]   x, x_sd [b][J][I][half][c][n][4 rows]   scratch G row [b][J][half][c][n][4 cols]
    const int64_t DN8 = (int64_t)Dm * N * 8;
    const int64_t DN4 = DN8 / 2;
    // Addressed as a wave-uniform base (batch image, tile) plus one 32-bit byte offset per lane, laneB: one register for
    // all of them across the tile loop instead of a 64-bit pointer per array.
    const uint32_t laneB = (uint32_t)(cc * N + nn) * 16u;              // the lane's four floats inside a half tile
    const char *xv = (const char *)(f.x_v + (int64_t)b * geo.nCY * geo.nCX * DN8);
    const char *xh = (const char *)(f.x + (int64_t)b * geo.nCX * geo.nCY * DN8);
    const char *xs = (const char *)(f.x_sd + (int64_t)b * geo.nCX * geo.nCY * DN8);
    auto ck4 = [&](const char *tile, int64_t floats) __attribute__((always_inline)) {   // 16 bytes of this lane, `floats` into the tile
        return *(const float4 *)(tile + floats * 4 + laneB);
    };
    // hand-over between blocks (pipelined schedules): [J][pair k][c][n][2], so that a wave's 8-byte
    // coherent accesses cover whole lines too (the lane's offset there is half of laneB)
    const int64_t DN2 = (int64_t)Dm * N * 2;
    char *gdown = (char *)((float *)p.workspace + nSync + (int64_t)b * geo.nCX * DN8);
    const uint32_t laneG = PIPE ? laneB >> 1 : laneB;

    const float *myDl = sDl + cl * DLP;
    const float *myDu = sDu + cl * PCH;
    const float *myDo = sDo + cl * PCH;
    const float *myB = sB + n * NSTR;
    const float *myC = sC + n * NSTR;
    float *mydB = sdB + wave * NP * NSD + n * NSD;
    float *mydC = sdC + wave * NP * NSD + n * NSD;
    const int qrow = (tid & 63) >> 4;               // 16-lane row of this lane inside its wave

    // ---- register staging of one tile's raw inputs (loaded at the start of the tile, then committed to LDS)
    float qb[VEC ? 1 : NBC], qc[VEC ? 1 : NBC], qdl[VEC ? 1 : NPX], qu[VEC ? 1 : NPX], qdo[VEC ? 1 : NPX], qh[VEC ? 1 : NHK];
    Raw4<T> vb, vc, vdl[VEC ? NCH : 1], vu[VEC ? NCH : 1];     // (VEC) one chunk of B and C, NCH chunks of delta, u, dout
    uint32_t vdo[VEC ? NCH : 1][4];
    uint32_t vh[VEC ? NHV : 1];
    // (VEC) halo cell k of this thread: cells 0-7 the row above, 8-15 the row below, 16-23 the column to the left
    auto halo_cell = [&](int hidx, int &rr, int &jj) {
        if (hidx < 8) { rr = -1; jj = hidx; }
        else if (hidx < 16) { rr = TE; jj = hidx - 8; }
        else { rr = hidx - 16; jj = -1; }
    };
    auto prefetch = [&](int I, int J) {
        const int r0 = (SND_TILE_ABLATE & 2) ? 0 : I * TE, j0 = (SND_TILE_ABLATE & 2) ? 0 : J * TE;
        // The thread's element maps are re-derived here from an opaque copy of the thread id, so that
        // they are a few integer ops per tile instead of dozens of registers kept live across the tile.
        SND_THREAD_MAPS(NP);
        if constexpr (VEC) {
            // loads are always in bounds (clamped coordinates); commit() zeroes what lies outside the plane.
            // Chunk q of a tile = row q / 2, columns 4 * (q % 2) .. + 3; under a mirrored column order the same four
            // memory columns in reverse (the chunk then starts at the memory column of its last scan column).
            auto chunk_off = [&](int q, int hB, int esz) {
                const int row = min(r0 + (q >> 1), H - 1), col = min(j0 + (q & 1) * 4, W - 4);
                return (uint32_t)mad24(mrow(row), hB, mcol(col + (fh ? 3 : 0)) * esz);
            };
            uint32_t z_ = 0;                        // (timing studies) what a load that is switched off leaves in its registers
            if (SND_TILE_ABLATE & 112) asm volatile("v_mov_b32 %0, 0x3e000000" : "=v"(z_));
            if (SND_TILE_ABLATE & 16) {
                for (int e = 0; e < (int)sizeof(T); ++e) { vb.w[e] = z_; vc.w[e] = z_; }
            } else {
                const int sn = min(t_ >> 4, N - 1), q = t_ & 15;
                ldraw4_b(vb, (const T *)((const char *)Bb + sn * BsB), chunk_off(q, BhB, ESZ));
                ldraw4_b(vc, (const T *)((const char *)Cb + sn * CsB), chunk_off(q, ChB, ESZ));
            }
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const int q = n + NP * k;
                if (SND_TILE_ABLATE & 32) {
                    for (int e = 0; e < (int)sizeof(T); ++e) { vdl[k].w[e] = z_; vu[k].w[e] = z_; }
                    for (int e = 0; e < 4; ++e) vdo[k][e] = z_;
                    continue;
                }
                ldraw4_b(vdl[k], db, cDb + chunk_off(q, DhB, ESZ));
                ldraw4_b(vu[k], ub, cUb + chunk_off(q, UhB, ESZ));
                const char *src = (const char *)dob + (cDob + chunk_off(q, DohB, esz_do));
                if (sizeof(T) == 4 || sh_do == 2) {
                    const uint4 v = *(const uint4 *)src;
                    vdo[k][0] = v.x; vdo[k][1] = v.y; vdo[k][2] = v.z; vdo[k][3] = v.w;
                } else {
                    const uint2 v = *(const uint2 *)src;
                    vdo[k][0] = v.x; vdo[k][1] = v.y;
                }
            }
#pragma unroll
            for (int k = 0; k < NHV; ++k) {
                int rr, jj;
                halo_cell(n + NP * k, rr, jj);
                const int row = min(max(r0 + rr, 0), H - 1), col = min(max(j0 + jj, 0), W - 1);
                if (SND_TILE_ABLATE & 64) { vh[k] = z_; continue; }
                vh[k] = ldraw_b(db, cDb + mad24(mrow(row), DhB, mcol(col) * ESZ));
            }
            return;
        }
        // loads are always in bounds (clamped coordinates); values outside the plane become zero
        {
            const int row = r0 + pr, col = j0 + pj;
            const bool in = pr < TE && pj < TE && row < H && col < W;
            const int mr = mrow(min(row, H - 1)), mcB = mcol(min(col, W - 1)) * ESZ;
            const uint32_t ob = mad24(mr, BhB, mcB), oc = mad24(mr, ChB, mcB);
#pragma unroll
            for (int k = 0; k < NBC; ++k) {
                const int sn = wave_u + WPB * k, sc = min(sn, N - 1);       // scalar: folded into the base
                const float vb_ = ldg_b((const T *)((const char *)Bb + sc * BsB), ob);
                const float vc_ = ldg_b((const T *)((const char *)Cb + sc * CsB), oc);
                qb[k] = (in && sn < N) ? vb_ : 0.f;
                qc[k] = (in && sn < N) ? vc_ : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < NPX; ++k) {
            const int pp = n + NP * k;
            const int row = r0 + (pp >> 3), col = j0 + (pp & 7);
            const bool ok = cvalid && (pp >> 3) < TE && (pp & 7) < TE && row < H && col < W;
            const int mr = mrow(min(row, H - 1)), mc = mcol(min(col, W - 1));
            const float vd = ldg_b(db, cDb + mad24(mr, DhB, mc * ESZ)), vu_ = ldg_b(ub, cUb + mad24(mr, UhB, mc * ESZ));
            const float vo = ld_f32_b(dob, cDob + mad24(mr, DohB, mc << sh_do), p.dout_dtype);
            qdl[k] = ok ? vd : 0.f;
            qu[k] = ok ? vu_ : 0.f;
            qdo[k] = ok ? vo : 0.f;
        }
#pragma unroll
        for (int k = 0; k < NHK; ++k) {   // the ring of halo cells around the tile in the delta' grid
            const int hidx = n + NP * k;
            int rr, jj;
            if (hidx < TE + 2) { rr = 0; jj = hidx; }
            else if (hidx < 2 * TE + 4) { rr = TE + 1; jj = hidx - (TE + 2); }
            else if (hidx < 3 * TE + 4) { rr = hidx - (2 * TE + 3); jj = 0; }
            else { rr = hidx - (3 * TE + 3); jj = TE + 1; }
            const int row = r0 - 1 + rr, col = j0 - 1 + jj;
            const bool ok = cvalid && hidx < NHALO && row >= 0 && row < H && col >= 0 && col < W;
            const float vd = ldg_b(db, cDb + mad24(mrow(min(max(row, 0), H - 1)), DhB, mcol(min(max(col, 0), W - 1)) * ESZ));
            qh[k] = ok ? vd : 0.f;
        }
    };
    auto commit = [&](int I, int J) {
        SND_THREAD_MAPS(NP);
        if constexpr (VEC) {
            const int r0 = I * TE, j0 = J * TE;
            auto flip4 = [&](float (&v)[4]) {                     // memory order -> scan order under a mirrored column order
                if (fh) { const float a0 = v[0], a1 = v[1]; v[0] = v[3]; v[1] = v[2]; v[2] = a1; v[3] = a0; }
            };
            {
                const int sn = t_ >> 4, q = t_ & 15;
                const bool ok = sn < N && r0 + (q >> 1) < H && j0 + (q & 1) * 4 < W;
                float b4[4], c4[4];
                raw4_to_f32(vb, b4); raw4_to_f32(vc, c4);
                flip4(b4); flip4(c4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { b4[e] = ok ? b4[e] : 0.f; c4[e] = ok ? c4[e] : 0.f; }
                *(float4 *)(sB + sn * NSTR + q * 4) = make_float4(b4[0], b4[1], b4[2], b4[3]);
                *(float4 *)(sC + sn * NSTR + q * 4) = make_float4(c4[0], c4[1], c4[2], c4[3]);
            }
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const int q = n + NP * k;
                const bool ok = cvalid && r0 + (q >> 1) < H && j0 + (q & 1) * 4 < W;
                float d4[4], u4[4], o4[4], dl4[4], du4[4], sg4[4];
                raw4_to_f32(vdl[k], d4); raw4_to_f32(vu[k], u4);
                if (sizeof(T) == 4 || sh_do == 2) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) o4[e] = __builtin_bit_cast(float, vdo[k][e]);
                } else {
                    Raw4<T> t4;
                    t4.w[0] = vdo[k][0]; t4.w[sizeof(T) == 4 ? 0 : 1] = vdo[k][1];
                    raw4_to_f32(t4, o4);
                }
                flip4(d4); flip4(u4); flip4(o4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float raw = (ok ? d4[e] : 0.f) + bias;
                    float dsp = 1.f;
                    dl4[e] = softplus ? softplus20(raw, dsp) : raw;
                    u4[e] = ok ? u4[e] : 0.f;
                    du4[e] = dl4[e] * u4[e];
                    o4[e] = ok ? wm * o4[e] : 0.f;
                    sg4[e] = dsp;
                }
                *(float4 *)(sDl + cl * DLP + ((q >> 1) + 1) * HG + DLO + (q & 1) * 4) = make_float4(dl4[0], dl4[1], dl4[2], dl4[3]);
                *(float4 *)(sDu + cl * PCH + q * 4) = make_float4(du4[0], du4[1], du4[2], du4[3]);
                *(float4 *)(sU + cl * PCS + q * 4) = make_float4(u4[0], u4[1], u4[2], u4[3]);
                *(float4 *)(sDo + cl * PCH + q * 4) = make_float4(o4[0], o4[1], o4[2], o4[3]);
                *(float4 *)(sSg + cl * PCS + q * 4) = make_float4(sg4[0], sg4[1], sg4[2], sg4[3]);
            }
#pragma unroll
            for (int k = 0; k < NHV; ++k) {
                const int hidx = n + NP * k;
                int rr, jj;
                halo_cell(hidx, rr, jj);
                const bool ok = cvalid && r0 + rr >= 0 && r0 + rr < H && j0 + jj >= 0 && j0 + jj < W;
                const float raw = (ok ? raw_to_f32((const T *)nullptr, vh[k]) : 0.f) + bias;
                float dsp;
                if (hidx < 24) sDl[cl * DLP + (rr + 1) * HG + DLO + jj] = softplus ? softplus20(raw, dsp) : raw;
            }
            return;
        }
#pragma unroll
        for (int k = 0; k < NBC; ++k) {
            const int sn = wave + WPB * k;
            sB[sn * NSTR + px] = qb[k];
            sC[sn * NSTR + px] = qc[k];
        }
#pragma unroll
        for (int k = 0; k < NPX; ++k) {
            const int pp = n + NP * k;
            const float raw = qdl[k] + bias;
            float dsp = 1.f;
            const float dl = softplus ? softplus20(raw, dsp) : raw;
            if (TE == 8 || ((pp >> 3) < TE && (pp & 7) < TE))     // slots beyond the tile belong to the halo ring
                sDl[cl * DLP + ((pp >> 3) + 1) * HG + DLO + (pp & 7)] = dl;
            sDu[cl * PCH + pp] = dl * qu[k];
            sU[cl * PCS + pp] = qu[k];
            sDo[cl * PCH + pp] = wm * qdo[k];
            sSg[cl * PCS + pp] = dsp;
        }
#pragma unroll
        for (int k = 0; k < NHK; ++k) {
            const int hidx = n + NP * k;
            int rr, jj;
            if (hidx < TE + 2) { rr = 0; jj = hidx; }
            else if (hidx < 2 * TE + 4) { rr = TE + 1; jj = hidx - (TE + 2); }
            else if (hidx < 3 * TE + 4) { rr = hidx - (2 * TE + 3); jj = 0; }
            else { rr = hidx - (3 * TE + 3); jj = TE + 1; }
            const float raw = qh[k] + bias;
            float dsp;
            if (hidx < NHALO && DLO - 1 + jj < HG)      // (the column right of an 8-column tile is never read)
                sDl[cl * DLP + rr * HG + DLO - 1 + jj] = softplus ? softplus20(raw, dsp) : raw;
        }
    };
#define DL(r, j) myDl[((r) + 1) * HG + DLO + (j)]
#define AEXP(r, j) EXPA(DL(r, j))
    // delta' of columns c0 .. c0+3 (c0 = 0 or 4) of tile row r (-1 .. 8): one aligned 16-byte read
    auto dl_row4 = [&](int r, int c0, float (&o)[4]) __attribute__((always_inline)) {
        const float4 v = *(const float4 *)(myDl + (r + 1) * HG + DLO + c0);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    };
#define EXPA(x) fast_exp2(fmaf((x), A2, ld))

    float dA_acc = 0.f, dec_acc = 0.f;              // per lane: sum delta'*da*a, sum da*a
    const bool want_decay = p.dA_decay != nullptr;  // the second sum is skipped when nobody reads it
    float dD_acc = 0.f, dbias_acc = 0.f;            // per thread, for its channel's staged pixels
    // Fused CrossMerge: weight * d(weight) = <weighted dout, result of the channel>.  The result is linear in u
    // (D*u plus a recurrence that is linear in B*delta'*u), so this inner product equals <du, u>: summed per pixel
    // beside dD, at no cost in the sweep.
    float dw_acc = 0.f;

    // dB, dC of a tile leave the block (summed over its channels) one tile late, from the partial sums that stay
    // in LDS until the next sweep: between the requests for the next tile's inputs and the wait for them, so that the
    // LDS reads and the address arithmetic of the flush fall under the latency of those loads (B=64, D=192, 56x56:
    // 1.290 -> 1.258 ms against the flush behind the wait, which -DSND_BWD_FLUSH_LATE restores for timing; with the
    // sums in front of the wait and the atomics behind it the eight values kept across the wait are spilled and
    // nothing more is gained, and the per-pixel epilogue moved to the same place gains nothing either).
    int pI = -1, pJ = 0;                            // the tile whose partial sums are still in LDS
    auto flush_bc = [&](int I_, int J_) __attribute__((always_inline)) {
        SND_THREAD_MAPS(NP);
        const int row = I_ * TE + pr, col = J_ * TE + pj;
        const bool in = pr < TE && pj < TE && row < H && col < W;
        const uint32_t o = mad24(mrow(row), W4, mcol(col) * 4);
#pragma unroll
        for (int k = 0; k < NBC; ++k) {
            const int sn = wave_u + WPB * k;                        // scalar: folded into the base
            float tb = 0.f, tc = 0.f;
#pragma unroll
            for (int w = 0; w < NPART; ++w) {
                tb += sdB[w * NP * NSD + sn * NSD + px];
                tc += sdC[w * NP * NSD + sn * NSD + px];
            }
            if (in && sn < N && !(SND_TILE_ABLATE & 1)) {
                glb_add((float *)((char *)dBg + sn * HW4 + o), tb);
                glb_add((float *)((char *)dCg + sn * HW4 + o), tc);
            } else if (SND_TILE_ABLATE & 1) {
                dbias_acc += tb + tc;               // keeps the values live
            }
        }
    };
    for (int I = I_hi; I >= I_lo; --I) {
        const int r0 = I * TE;
        float GR[kRows], GsR[kRows];                // G, Gs at the column right of the tile
        float aR[kRows];                            // a at that column (only ever multiplies G there)
        float GRc = 0.f;                            // G[r0+8][j0+8]
#pragma unroll
        for (int r = 0; r < kRows; ++r) { GR[r] = 0.f; GsR[r] = 0.f; aR[r] = 0.f; }
        if (SEG && seg > 0) {
            // a later column segment of the strip: G, Gs, a of the column right of it and the corner G come from the
            // block that swept the segment before (written in full before its count moved: see strip_stores_done)
            if (wave == 0) {
                int seen_ = 0;
                strip_wait(segdone + I, seg, seen_, sync, dead, geo.spinLimit SND_TRACE_PASS);
                if (dead && tid == 0) sDead = 1;
            }
            __syncthreads();
            const float *src = colstate + (tid << 1);
            const bool bad = lds_peek(&sDead) != 0;   // the wait timed out: poison everything downstream
#pragma unroll
            for (int r = 0; r < kRows; r += 2) {
                ld2_coherent(src + (r >> 1) * 512, GR[r], GR[r + 1]);
                ld2_coherent(src + (4 + (r >> 1)) * 512, GsR[r], GsR[r + 1]);
                ld2_coherent(src + (8 + (r >> 1)) * 512, aR[r], aR[r + 1]);
            }
            float pad_;
            ld2_coherent(src + 12 * 512, GRc, pad_);
            if (bad) {
                GRc = __builtin_nanf("");
#pragma unroll
                for (int r = 0; r < kRows; ++r) GR[r] = GsR[r] = __builtin_nanf("");
            }
        }

        for (int J = SEG ? J_hi : geo.nCX - 1; J >= (SEG ? J_lo : 0); --J) {
            const int j0 = J * TE;
            // ---- checkpoints and carried adjoints of this tile: requested first, so that they arrive
            // under the staging below instead of being waited for after the barrier
            float hu[kCkX], hlft[kRows], slft[kRows], hc = 0.f;   // h row above, h/s column to the left
            float Gd[kCkX];                                        // G of the row below
            if (I > 0) {
                const char *src = xv + ((SND_TILE_ABLATE & 8) ? 1 : ((int64_t)(I - 1) * geo.nCX + J)) * DN8 * 4;
                const float4 v0 = ck4(src, 0), v1 = ck4(src, DN4);
                hu[0] = v0.x; hu[1] = v0.y; hu[2] = v0.z; hu[3] = v0.w;
                hu[4] = v1.x; hu[5] = v1.y; hu[6] = v1.z; hu[7] = v1.w;
                if (J > 0)                          // last column of the tile on the left
                    hc = *(const float *)(src + (((TE - 1) >> 2) * DN4 + ((TE - 1) & 3) - DN8) * 4 + laneB);
            } else {
#pragma unroll
                for (int j = 0; j < kCkX; ++j) hu[j] = 0.f;
            }
            if (J > 0) {
                const char *sh_ = xh + ((SND_TILE_ABLATE & 8) ? 0 : ((int64_t)(J - 1) * geo.nCY + I)) * DN8 * 4;
                const char *ss_ = xs + ((SND_TILE_ABLATE & 8) ? 0 : ((int64_t)(J - 1) * geo.nCY + I)) * DN8 * 4;
                const float4 h0 = ck4(sh_, 0), h1 = ck4(sh_, DN4);
                const float4 s0 = ck4(ss_, 0), s1 = ck4(ss_, DN4);
                hlft[0] = h0.x; hlft[1] = h0.y; hlft[2] = h0.z; hlft[3] = h0.w;
                hlft[4] = h1.x; hlft[5] = h1.y; hlft[6] = h1.z; hlft[7] = h1.w;
                slft[0] = s0.x; slft[1] = s0.y; slft[2] = s0.z; slft[3] = s0.w;
                slft[4] = s1.x; slft[5] = s1.y; slft[6] = s1.z; slft[7] = s1.w;
            } else {
#pragma unroll
                for (int r = 0; r < kRows; ++r) { hlft[r] = 0.f; slft[r] = 0.f; }
            }
            // the adjoint row of the strip below: written by this block, or - first strip of a
            // pipelined band - by another block.  It is requested here if it is known to be there (own
            // rows; rows whose hand-over an earlier poll has already seen), else after the wait below.
            const bool handed = PIPE && I == I_hi && I + 1 < geo.nCY;
            const bool late = handed && __builtin_amdgcn_readfirstlane(lds_peek(&sSeen)) < geo.nCX - J;
            if (!late) {
                if (I + 1 < geo.nCY && lvalid) {
                    const char *src = gdown + (int64_t)J * DN8 * 4;
                    if (PIPE) {
#pragma unroll
                        for (int k = 0; k < kCkX; k += 2) ld2_coherent((const float *)(src + (k >> 1) * DN2 * 4 + laneG), Gd[k], Gd[k + 1]);
                    } else {
                        const float4 v0 = *(const float4 *)(src + laneG), v1 = *(const float4 *)(src + DN4 * 4 + laneG);
                        Gd[0] = v0.x; Gd[1] = v0.y; Gd[2] = v0.z; Gd[3] = v0.w;
                        Gd[4] = v1.x; Gd[5] = v1.y; Gd[6] = v1.z; Gd[7] = v1.w;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) Gd[j] = 0.f;
                }
            }
            prefetch(I, J);                         // no loads in flight across the register-hungry sweep
#ifndef SND_BWD_FLUSH_LATE
            if (pI >= 0) flush_bc(pI, pJ);          // the previous tile's dB, dC, under the latency of the loads just requested
            commit(I, J);
#else                                               // (timing study: the flush behind the wait, as it was; same results)
            commit(I, J);
            if (pI >= 0) flush_bc(pI, pJ);
#endif
            pI = I; pJ = J;
            // strip pipeline: the strip below must have handed over tile J.  One wave polls; the
            // others wait at the barrier.
            if (handed && wave == 0) {
                strip_wait(progress + I + 1, geo.nCX - J, seen, sync, dead, geo.spinLimit SND_TRACE_PASS);
                if (tid == 0) { sSeen = seen; if (dead) sDead = 1; }   // read at the top of later tiles
            }
            __syncthreads();
            // The sweep runs at a raised wave priority, everything else (loads, commit to LDS, per-pixel epilogue) at the
            // default: the two waves a SIMD holds belong to two blocks, and with equal priority they drift into the same
            // phase and stall together; with the wave that is in its dependent arithmetic chain preferred, the other's
            // memory phases fall into its gaps.  Measured (same box, backward ms): c1 1.332 -> 1.280, c2 0.339 -> 0.331,
            // c3 1.199 -> 1.181, c4 2.765 -> 2.664; priorities 1, 2, 3 alike, the reverse assignment half as much, a fixed
            // priority per block nothing.
            __builtin_amdgcn_s_setprio(3);

            if (late) {                             // only after the wait above
                if (I + 1 < geo.nCY && lvalid) {
                    const char *src = gdown + (int64_t)J * DN8 * 4;
#pragma unroll
                    for (int k = 0; k < kCkX; k += 2) ld2_coherent((const float *)(src + (k >> 1) * DN2 * 4 + laneG), Gd[k], Gd[k + 1]);
                } else {
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) Gd[j] = 0.f;
                }
            }
            if (handed && lds_peek(&sDead)) {   // the wait timed out: poison everything downstream
#pragma unroll
                for (int j = 0; j < kCkX; ++j) Gd[j] = __builtin_nanf("");
            }
            const float gd_old0 = Gd[0];            // G[r0+8][j0]: the corner of the tile on the left

            // The tile is swept as two 8x4 halves, right then left, so that only 32 values of h
            // are held at a time.  The right half starts from h, s at column 3, which a plain
            // forward pass over the left half provides first (that half is recomputed when it is
            // swept: 32 extra cell updates per tile buy about 60 registers).
            float hmid[kRows] = {}, smid[kRows] = {}, amid[kRows] = {};   // h, s, a at column 3
            {
                float aprev[4], hprev[4], dlr[4];
                dl_row4(-1, 0, dlr);
#pragma unroll
                for (int j = 0; j < 4; ++j) { aprev[j] = EXPA(dlr[j]); hprev[j] = hu[j]; }
                float diag0 = hc;
#pragma unroll
                for (int r = 0; r < TE; ++r) {
                    float al = AEXP(r, -1), left = hlft[r], sl = slft[r], diag = diag0;
                    diag0 = hlft[r];
                    dl_row4(r, 0, dlr);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float a = EXPA(dlr[j]);
                        const float bu = myB[r * kCkX + j] * myDu[r * kCkX + j];
                        const float up = hprev[j];
                        const float X = fmaf(-0.5f * (aprev[j] + al), diag, up);
                        const float h = fmaf(a, left + X, bu);
                        sl = fmaf(a, sl, bu);
                        hprev[j] = h;
                        diag = up; left = h; al = a; aprev[j] = a;
                    }
                    hmid[r] = left; smid[r] = sl; amid[r] = al;
                }
            }

            // One half: recompute h on rows 0..7, columns C0..C0+3, then sweep it bottom-right to
            // top-left.  top/corner: h of the row above; hL/sL: h, s of the column to the left;
            // GR/GsR (in/out): G, Gs of the column to the right, replaced by those of column C0;
            // GdH (in/out): G of the row below, replaced by G of row 0; gdiag0: G[8][C0+4].
            auto sweep_half = [&](auto C0_, const float *top, float corner, const float (&hL)[kRows],
                                  const float (&sL)[kRows], float *GdH, float gdiag0) {
                constexpr int C0 = decltype(C0_)::value;
                constexpr int HW = C0 == 0 ? 4 : TE - 4;        // columns of this half inside the tile
                float hT[kRows][4];
                // the left half keeps a of its first KA columns from this pass for the sweep (as many as
                // fit under 256 registers without spilling); everything else is recomputed there
                constexpr int KA = C0 == 0 ? (TE == 7 ? 4 : SND_KA8) : 0;
                float aT[KA ? kRows : 1][KA ? KA : 1];
                {
                    float aprev[4], hprev[4], dlr[4];
                    dl_row4(-1, C0, dlr);
#pragma unroll
                    for (int j = 0; j < HW; ++j) { aprev[j] = EXPA(dlr[j]); hprev[j] = top[j]; }
                    float diag0 = corner;
#pragma unroll
                    for (int r = 0; r < TE; ++r) {
                        float al = C0 == 0 ? AEXP(r, C0 - 1) : amid[r], left = hL[r], diag = diag0;
                        diag0 = hL[r];
                        dl_row4(r, C0, dlr);
#pragma unroll
                        for (int j = 0; j < HW; ++j) {
                            const float a = EXPA(dlr[j]);
                            const float bu = myB[r * kCkX + C0 + j] * myDu[r * kCkX + C0 + j];
                            const float up = hprev[j];
                            const float X = fmaf(-0.5f * (aprev[j] + al), diag, up);
                            const float h = fmaf(a, left + X, bu);
                            hT[r][j] = h;
                            if (j < KA) aT[r][j] = a;
                            hprev[j] = h;
                            diag = up; left = h; al = a; aprev[j] = a;
                        }
                    }
                }
                float adn[4];
                float Gd8 = gdiag0;
                {
                    float dlr[4];
                    dl_row4(TE, C0, dlr);
#pragma unroll
                    for (int j = 0; j < HW; ++j) adn[j] = EXPA(dlr[j]);
                }
                // The five LDS operands of a row (delta', B, C, delta'*u, dout; 16 bytes each) are requested one row ahead.
                // With 7x7 tiles, 16 states and whole-plane blocks the request sits behind the row's cell updates and in front of its
                // cross-lane sums (the registers of the row just finished are free there, and the reads complete under
                // the sums: 64 x 768 channels of 14x14, bf16, 0.347 -> 0.336 ms); every other variant has no register
                // left for that (12 to 16 spilled, nothing gained) and requests the next row behind the sums.
                constexpr bool ROWPF = TE == 7 && NP == 16 && !PIPE;
                float4 nD4, nB4, nC4, nU4, nO4;
                auto request_row = [&](int r) __attribute__((always_inline)) {
                    nD4 = *(const float4 *)(myDl + (r + 1) * HG + DLO + C0);
                    nB4 = *(const float4 *)(myB + r * kCkX + C0);
                    nU4 = *(const float4 *)(myDu + r * kCkX + C0);
                    nC4 = *(const float4 *)(myC + r * kCkX + C0); nO4 = *(const float4 *)(myDo + r * kCkX + C0);
                };
                request_row(TE - 1);
#pragma unroll
                for (int r = TE - 1; r >= 0; --r) {
                    __builtin_amdgcn_sched_barrier(0);
                    float arow[5], s[4], buv[4];
                    const float dlr[4] = {nD4.x, nD4.y, nD4.z, nD4.w};
#pragma unroll
                    for (int j = 0; j < HW; ++j) arow[j] = j < KA ? aT[KA ? r : 0][j < KA ? j : 0] : EXPA(dlr[j]);
                    arow[HW] = aR[r];
                    const float aB[4] = {nB4.x, nB4.y, nB4.z, nB4.w}, aC[4] = {nC4.x, nC4.y, nC4.z, nC4.w};
                    const float aU[4] = {nU4.x, nU4.y, nU4.z, nU4.w}, aO[4] = {nO4.x, nO4.y, nO4.z, nO4.w};
                    {
                        float sp = sL[r];
#pragma unroll
                        for (int j = 0; j < HW; ++j) {
                            buv[j] = aB[j] * aU[j];
                            sp = fmaf(arow[j], sp, buv[j]);
                            s[j] = sp;
                        }
                    }
                    float Gr = GR[r], Gsr = GsR[r], Gdiag = Gd8;
                    float q[4] = {}, pp_[4] = {}, vB[4] = {}, vC[4] = {}, dsum[4] = {};
#pragma unroll
                    for (int j = HW - 1; j >= 0; --j) {
                        const float dov = aO[j];
                        const float Bv = aB[j], Cv = aC[j];
                        const float duv = aU[j];
                        const float bu = buv[j];
                        const float dyC = dov * Cv;
                        const float a = arow[j];
                        const float g_ = fmaf(-0.5f * (arow[j + 1] + adn[j]), Gdiag, dyC + Gr + GdH[j]);
                        const float gs = Gsr - dyC;
                        const float dbu = fmaf(0.25f, dyC, g_ + gs);
                        const float h_l = (j == 0) ? hL[r] : hT[r][j - 1 < 0 ? 0 : j - 1];
                        const float h_u = (r == 0) ? top[j] : hT[r - 1 < 0 ? 0 : r - 1][j];
                        // g(h - bu) + gs(s - bu) = g(h - s) + (g + gs)(s - bu)
                        const float hs = hT[r][j] - s[j], sb = s[j] - bu;
                        const float cross = fmaf(GdH[j], h_l, Gr * h_u);
                        const float da = fmaf(-0.5f * a, cross, fmaf(g_, hs, (g_ + gs) * sb));
                        dA_acc = fmaf(dlr[j], da, dA_acc);
                        dsum[j] = da;
                        const float Gn = a * g_;
                        Gdiag = GdH[j];
                        GdH[j] = Gn;
                        Gr = Gn;
                        Gsr = a * gs;
                        q[j] = dbu * Bv;                           // per-pixel terms, summed over states below
                        pp_[j] = Av * da;
                        vB[j] = dbu * duv;                         // dB, dC contributions
                        vC[j] = dov * fmaf(0.25f, bu, hs);
                    }
                    // The two running sums are pinned to their row: left to itself the compiler sinks the whole chain of
                    // multiply-adds to the end of the tile and keeps delta' and da of all 64 cells in registers until then.
                    if (want_decay) dec_acc += (dsum[0] + dsum[1]) + (dsum[2] + dsum[3]);
                    if (ROWPF) {
                        if (r > 0) request_row(r - 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (NP == 16) {
                        // sums over the channel's 16 states: quads 0,1 of the lane group end with
                        // q[0..1], q[2..3], quads 2,3 with pp_[0..1], pp_[2..3]
                        group_scatter8(q[0], q[1], q[2], q[3], pp_[0], pp_[1], pp_[2], pp_[3]);
                        if ((n & 3) == 0) {
                            float *dst = ((n & 8) ? sP : sQ) + cl * PCH + r * kCkX + C0 + ((n >> 1) & 2);
                            *(float2 *)dst = make_float2(q[0], q[1]);
                        }
                    } else {
                        group_sum4<NP>(q[0], q[1], q[2], q[3]);
                        group_sum4<NP>(pp_[0], pp_[1], pp_[2], pp_[3]);
                        if (n == 0) {
                            *(float4 *)(sQ + cl * PCH + r * kCkX + C0) = make_float4(q[0], q[1], q[2], q[3]);
                            *(float4 *)(sP + cl * PCH + r * kCkX + C0) = make_float4(pp_[0], pp_[1], pp_[2], pp_[3]);
                        }
                    }
                    {
                        // sum over the wave's channels: lane bits 4-5 by a swap reduce-scatter (the
                        // 16-lane row q ends with column C0+q), bits 3 and 2 (8- and 4-lane layouts) by row rotates
                        rows_scatter4x2(vB[0], vB[1], vB[2], vB[3], vC[0], vC[1], vC[2], vC[3]);
                        float tb = vB[0], tc = vC[0];
                        if (NP <= 8) { tb += dpp_mov<0x128>(tb); tc += dpp_mov<0x128>(tc); }   // row_ror:8
                        if (NP <= 4) { tb += dpp_mov<0x124>(tb); tc += dpp_mov<0x124>(tc); }   // row_ror:4
                        if ((tid & (16 - NP)) == 0) {
                            mydB[r * kCkX + C0 + qrow] = tb;
                            mydC[r * kCkX + C0 + qrow] = tc;
                        }
                    }
                    if (!ROWPF && r > 0) request_row(r - 1);
                    Gd8 = GR[r];                    // G[r][C0+4]: diagonal neighbour for the row above
                    GR[r] = Gr;                     // G[r][C0]: right neighbour for the half on the left
                    GsR[r] = Gsr;
                    aR[r] = arow[0];
#pragma unroll
                    for (int j = 0; j < HW; ++j) adn[j] = arow[j];
                }
            };
            const float gd_old4 = Gd[4];            // G[r0+8][j0+4]: corner of the left half
            sweep_half(std::integral_constant<int, 4>{}, hu + 4, hu[3], hmid, smid, Gd + 4, GRc);
            sweep_half(std::integral_constant<int, 0>{}, hu, hc, hlft, slft, Gd, gd_old4);
            GRc = gd_old0;
            const bool hands_over = PIPE && I == I_lo && I > 0;   // top strip of a band: another block takes the row
            if (I > 0 && lvalid) {                  // adjoint row for the strip above
                char *dst = gdown + (int64_t)J * DN8 * 4;
                if (PIPE) {
#pragma unroll
                    for (int k = 0; k < kCkX; k += 2) st2_coherent((float *)(dst + (k >> 1) * DN2 * 4 + laneG), Gd[k], Gd[k + 1]);
                } else {
                    *(float4 *)(dst + laneG) = make_float4(Gd[0], Gd[1], Gd[2], Gd[3]);
                    *(float4 *)(dst + DN4 * 4 + laneG) = make_float4(Gd[4], Gd[5], Gd[6], Gd[7]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            if (hands_over) strip_stores_done();
            __syncthreads();
            if (hands_over) strip_signal(progress + I);   // tile J is handed over to the strip above

            // ---- once per pixel: du, ddelta (thread that staged the pixel), dD, ddelta_bias
            {
            SND_THREAD_MAPS(NP);
            if constexpr (VEC) {
#pragma unroll
                for (int k = 0; k < NCH; ++k) {
                    const int q = n + NP * k;
                    const int row = r0 + (q >> 1), col = j0 + (q & 1) * 4;
                    const float4 q4 = *(const float4 *)(sQ + cl * PCH + q * 4), p4 = *(const float4 *)(sP + cl * PCH + q * 4);
                    const float4 l4 = *(const float4 *)(sDl + cl * DLP + ((q >> 1) + 1) * HG + DLO + (q & 1) * 4);
                    const float4 u4 = *(const float4 *)(sU + cl * PCS + q * 4), o4 = *(const float4 *)(sDo + cl * PCH + q * 4);
                    const float4 g4 = *(const float4 *)(sSg + cl * PCS + q * 4);
                    const float aq[4] = {q4.x, q4.y, q4.z, q4.w}, ap[4] = {p4.x, p4.y, p4.z, p4.w}, al[4] = {l4.x, l4.y, l4.z, l4.w};
                    const float au[4] = {u4.x, u4.y, u4.z, u4.w}, ao[4] = {o4.x, o4.y, o4.z, o4.w}, ag[4] = {g4.x, g4.y, g4.z, g4.w};
                    float duv[4], ddl[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        duv[e] = fmaf(Dv, ao[e], al[e] * aq[e]);
                        ddl[e] = fmaf(au[e], aq[e], ap[e]) * ag[e];
                    }
                    if (cvalid && row < H && col < W) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            dD_acc = fmaf(ao[e], au[e], dD_acc);
                            dw_acc = fmaf(duv[e], au[e], dw_acc);
                            dbias_acc += ddl[e];
                        }
                        if (fh) {                   // scan order -> memory order
                            const float a0 = duv[0], a1 = duv[1], b0 = ddl[0], b1 = ddl[1];
                            duv[0] = duv[3]; duv[1] = duv[2]; duv[2] = a1; duv[3] = a0;
                            ddl[0] = ddl[3]; ddl[1] = ddl[2]; ddl[2] = b1; ddl[3] = b0;
                        }
                        const uint32_t o = cGb + mad24(mrow(row), WB, mcol(col + (fh ? 3 : 0)) * ESZ);
                        if (!(SND_TILE_ABLATE & 4)) {
                            stg4_b(dub, o, duv);
                            stg4_b(ddb, o, ddl);
                        } else {
                            dD_acc += duv[0] + ddl[0];  // keeps the values live
                        }
                    }
                }
            } else {
#pragma unroll
            for (int k = 0; k < NPX; ++k) {
                const int pp = n + NP * k;
                const int row = r0 + (pp >> 3), col = j0 + (pp & 7);
                const float qv = sQ[cl * PCH + pp], pv = sP[cl * PCH + pp];
                const float dl = sDl[cl * DLP + ((pp >> 3) + 1) * HG + DLO + (pp & 7)];
                const float uv = sU[cl * PCS + pp], dov = sDo[cl * PCH + pp], sg = sSg[cl * PCS + pp];
                const float duv = fmaf(Dv, dov, dl * qv);
                const float ddl = fmaf(uv, qv, pv) * sg;
                if (cvalid && (pp >> 3) < TE && (pp & 7) < TE && row < H && col < W) {
                    dD_acc = fmaf(dov, uv, dD_acc);
                    dw_acc = fmaf(duv, uv, dw_acc);
                    dbias_acc += ddl;
                    const uint32_t o = cGb + mad24(mrow(row), WB, mcol(col) * ESZ);
                    if (!(SND_TILE_ABLATE & 4)) {
                        stg_b(dub, o, duv);
                        stg_b(ddb, o, ddl);
                    } else {
                        dD_acc += duv;              // keeps the values live
                    }
                }
            }
            }
            }
        }
        if (SEG && seg + 1 < geo.nSeg) {
            // hand the carried column state to the block of the strip's next segment: stores, each wave waits for its
            // own to complete, block barrier, then one thread moves the strip's count of finished segments
            float *dst = colstate + (tid << 1);
#pragma unroll
            for (int r = 0; r < kRows; r += 2) {
                st2_coherent(dst + (r >> 1) * 512, GR[r], GR[r + 1]);
                st2_coherent(dst + (4 + (r >> 1)) * 512, GsR[r], GsR[r + 1]);
                st2_coherent(dst + (8 + (r >> 1)) * 512, aR[r], aR[r + 1]);
            }
            st2_coherent(dst + 12 * 512, GRc, 0.f);
            strip_stores_done();
            __syncthreads();
            strip_signal(segdone + I);
        }
    }
    if (pI >= 0) flush_bc(pI, pJ);
#undef DL
#undef AEXP
#undef EXPA

#ifdef SND_PIPE_TRACE
    if (PIPE && threadIdx.x == 0) { trace_[1] = (int)wall_clock64(); trace_[2] = trace_wait_; }
#endif
    // ---- per-lane / per-channel sums leave the kernel
    if (lvalid) glb_add(p.dA + (int64_t)c * N + n, dA_acc);
    dD_acc = group_sum<NP>(dD_acc);
    dbias_acc = group_sum<NP>(dbias_acc);
    if (n == 0 && cvalid) {
        if (p.dD) glb_add(p.dD + c, dD_acc);
        if (p.ddelta_bias) glb_add(p.ddelta_bias + c, dbias_acc);
    }
    if (merge && p.dmerge) {
        dw_acc = group_sum<NP>(dw_acc);
        if (n == 0 && cvalid) glb_add(p.dmerge + c, dw_acc);
    }
    if (p.dA_decay) {
        float v = lvalid ? dec_acc : 0.f;
        v = group_sum<16>(v);
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        if ((tid & 63) == 0) sRed[wave] = v;
        __syncthreads();
        if (tid == 0) {
            float t = 0.f;
            for (int w = 0; w < WPB; ++w) t += sRed[w];
            glb_add(p.dA_decay, t / f.A_decay[0]);
        }
    }
}

// Dynamic LDS of one backward block (more than the 64 KB a kernel gets without asking).
template <int NP> constexpr size_t bwd_lds_bytes() {
    constexpr int PCH = kTile + (NP == 16 ? 8 : 4), PCS = kTile + NP, NSD = NP == 16 ? kTile + 2 : kTile + 4;
    return sizeof(float) * (2 * NP * (kTile + 4) + 2 * (NP / 4) * NP * NSD + 16 * 120 + 16 * (4 * PCH + 2 * PCS) + 4 + NP / 4);
}
// Raise the dynamic LDS limit of every backward instantiation of one input dtype on the current device.
// hipFuncSetAttribute is not stream-ordered and must not run under a stream capture, which is why it is
// done once per device at set-up and not inside the launch path.
template <typename T, int NP, int TE, bool VEC> static bool configure_bwd_one() {
    const int lds = (int)bwd_lds_bytes<NP>();
    if (NP == 16 && hipFuncSetAttribute((const void *)bwd_kernel<T, NP, true, TE, VEC, NP == 16>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return false;
    return hipFuncSetAttribute((const void *)bwd_kernel<T, NP, true, TE, VEC>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess &&
           hipFuncSetAttribute((const void *)bwd_kernel<T, NP, false, TE, VEC>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) == hipSuccess;
}
template <typename T> int configure_bwd_t() {
    const bool ok = configure_bwd_one<T, 16, 8, false>() && configure_bwd_one<T, 16, 7, false>() && configure_bwd_one<T, 8, 8, false>() &&
                    configure_bwd_one<T, 8, 7, false>() && configure_bwd_one<T, 4, 8, false>() && configure_bwd_one<T, 4, 7, false>() &&
                    configure_bwd_one<T, 16, 8, true>() && configure_bwd_one<T, 8, 8, true>() && configure_bwd_one<T, 4, 8, true>();
    return ok ? SND_OK : SND_ERR_LAUNCH;
}

// Whether a call can stage four columns per access (bwd_kernel's VEC): every row of every tensor the staging touches
// must start on a four-element boundary (16 bytes of fp32, 8 bytes of 16-bit values), and so must the rows of the dense
// du / ddelta; a state's plane of B / C must lie within 2^31 bytes of the first (the state offset is per lane there).
inline bool vec4_ok(const void *ptr, int esz, std::initializer_list<int64_t> strides) {
    if (((uintptr_t)ptr & (uintptr_t)(4 * esz - 1)) != 0) return false;
    for (int64_t s : strides)
        if (s % 4 != 0) return false;
    return true;
}
inline bool bwd_vec_ok(const snd_bwd_params &p) {
    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int e = sh.in_dtype == SND_F32 ? 4 : 2, eo = p.dout_dtype == SND_F32 ? 4 : 2;
    if (sh.ncols % 4 != 0) return false;
    const int64_t span = (int64_t)(sh.dstate - 1) * e;
    if (span * f.B_dstate_stride + (int64_t)sh.nrows * f.B_h_stride * e >= ((int64_t)1 << 31) ||
        span * f.C_dstate_stride + (int64_t)sh.nrows * f.C_h_stride * e >= ((int64_t)1 << 31))
        return false;
    return vec4_ok(f.u, e, {f.u_batch_stride, f.u_d_stride, f.u_h_stride}) &&
           vec4_ok(f.delta, e, {f.delta_batch_stride, f.delta_d_stride, f.delta_h_stride}) &&
           vec4_ok(f.B, e, {f.B_batch_stride, f.B_group_stride, f.B_dstate_stride, f.B_h_stride}) &&
           vec4_ok(f.C, e, {f.C_batch_stride, f.C_group_stride, f.C_dstate_stride, f.C_h_stride}) &&
           vec4_ok(p.dout, eo, {p.dout_batch_stride, p.dout_d_stride, p.dout_h_stride}) &&
           vec4_ok(p.du, e, {}) && vec4_ok(p.ddelta, e, {});
}

template <typename T, int NP, int TE, bool VEC>
static int launch_bwd_te(const snd_bwd_params &p, const Geo &geo, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    const int rg = sh.dim / sh.n_groups;
    const int nChunks = (rg + 15) / 16;
    const int64_t nPC = (int64_t)sh.batch * sh.n_groups * nChunks;
    constexpr size_t lds = bwd_lds_bytes<NP>();
    const int bands = bwd_band_count(p.f.schedule, (int64_t)sh.batch * sh.n_groups, nChunks, geo.nCY, p.workspace, sh.dstate, geo.nCX);   // 0: one block per plane chunk
    const bool pipe = bands > 0;
    // the dynamic LDS limit of these kernels is raised by snd_init() / on the first launch on a device
    if (int st = ensure_device_ready(); st != SND_OK) return st;
    if (pipe) {
        if (nPC * geo.nCY >= (int64_t)1 << 31) return SND_ERR_SHAPE;
        if (zero_words((int *)p.workspace, sync_words(nPC, geo.nCY), stream) != SND_OK) return SND_ERR_LAUNCH;
        Geo gb = geo;
        gb.spinLimit = spin_limit();
        gb.nBands = bands;
        gb.nQueues = job_queues(sh.batch * sh.n_groups);
        // one strip per job and more strips than block slots: the strips may be cut into column segments (the plan
        // has sized the workspace for their carried state)
        if (bands == geo.nCY && NP == 16) gb.nSeg = strip_segments(nPC, geo.nCY, geo.nCX, bwd_slots(sh.dstate), gb.nQueues);
        gb.segTiles = geo.nCX / gb.nSeg;
        if (nPC * bands * gb.nSeg >= (int64_t)1 << 31) return SND_ERR_SHAPE;
        if (NP == 16 && gb.nSeg > 1)
            hipLaunchKernelGGL((bwd_kernel<T, NP, true, TE, VEC, NP == 16>), dim3((int)(nPC * bands * gb.nSeg)), dim3(16 * NP), lds, stream, p, gb);
        else
            hipLaunchKernelGGL((bwd_kernel<T, NP, true, TE, VEC>), dim3((int)(nPC * bands)), dim3(16 * NP), lds, stream, p, gb);
    } else {
        const int grid = xcd_grid(sh.batch * sh.n_groups, nChunks);
        hipLaunchKernelGGL((bwd_kernel<T, NP, false, TE, VEC>), dim3(grid), dim3(16 * NP), lds, stream, p, geo);
    }
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T, int NP>
static int launch_bwd_np(const snd_bwd_params &p, hipStream_t stream) {
    Geo geo = make_geo(p.f.shape.nrows, p.f.shape.ncols);
    geo.tag = state_tag(p.f.x_sd, p.f.shape);
    if (geo.te == 7) return launch_bwd_te<T, NP, 7, false>(p, geo, stream);
    return bwd_vec_ok(p) ? launch_bwd_te<T, NP, 8, true>(p, geo, stream) : launch_bwd_te<T, NP, 8, false>(p, geo, stream);
}

// One instantiation per input dtype, each in its own translation unit.
template <typename T>
int launch_bwd_t(const snd_bwd_params &p, hipStream_t stream) {
    const int N = p.f.shape.dstate;
    return N > 8 ? launch_bwd_np<T, 16>(p, stream) : N > 4 ? launch_bwd_np<T, 8>(p, stream) : launch_bwd_np<T, 4>(p, stream);
}

}  // namespace snd
