// Backward kernel of the 2D-CrossScan selective scan for one to four states per channel (gfx950):
// the row-segment wavefront, run in reverse.
//
// Same gradients as snd_bwd_kernel.h (reference: selective_scan_bwd_kernel_oflex.cuh:91-902).  With
// G = a*g, Gs = a*gs and every out-of-range term zero, per (batch, channel, state) plane:
//     g[i,j]  = dout*C + G[i,j+1] + G[i+1,j] - 0.5*(a[i,j+1] + a[i+1,j])*G[i+1,j+1]
//     gs[i,j] = -dout*C + Gs[i,j+1]
//     dbu     = g + gs + 0.25*dout*C
//     da*a    = g*(h - bu) + gs*(s - bu) - 0.5*a*(G[i+1,j]*h[i,j-1] + G[i,j+1]*h[i-1,j])
// and from these du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay as listed in snd_bwd_kernel.h.
//
// Mapping as in snd_wave_fwd_kernel.h: a block per (batch, channel), a wave per 64-column row segment, the
// states in registers.  Along a row the adjoint is first order towards the left,
//     G_j = a_j*G_{j+1} + a_j*z_j,   z_j = dout*C + G[i+1,j] - 0.5*(a[i,j+1] + a[i+1,j])*G[i+1,j+1],
// so a wave resolves a row with one DPP scan, exactly like the forward - provided its lanes run against
// the columns.  Every load, store and the whole adjoint sweep therefore use the mirrored order (lane l owns
// the columns that lane 63 - l owns in the forward, and walks them downwards); only the recomputation of h and
// s, which runs with the columns, sees its inputs and leaves its results through a lane reversal (ds_bpermute:
// a register crossbar move, no LDS memory).
// A wave handles its segment band by band (R rows), bottom band first: recompute h, s of the band's rows
// from the forward's checkpoints (row above the band from x_v, what entered the segment on every row from
// x / x_sd: no wave waits for another here), then sweep the band's rows bottom-up.  The sweep needs G, Gs, a
// of the segment on the right at its first column: wave w runs one band behind wave w+1 and finds them in
// LDS (one block barrier per band, no polling).  dB, dC leave as one global atomic per element and channel
// (a wave-wide instruction covers 256 consecutive bytes), du / ddelta as whole row segments.
#pragma once
#include <initializer_list>
#include <type_traits>
#include "snd_device.h"

// Timing studies only (-DSND_WAVE_ABLATE=<bits>, results wrong): 64 no dB / dC atomics, 128 no du / ddelta stores,
// 256 (column groups) nothing left for the group on the left, 512 nothing taken from the group on the right.
#ifndef SND_WAVE_ABLATE
#define SND_WAVE_ABLATE 0
#endif

namespace snd {

constexpr int kWaveShareWaves = 8;                   // waves of a block whose channels share their dB / dC atomics

__device__ __forceinline__ void wave_glb_add(float *p, float v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// EVEN: the plane is a whole number of bands high and of 64-lane segments wide.  No row of a band and no lane is then
// skipped, so no branch surrounds the stores and atomics of a row: every band issues the same memory instructions on
// every path, and the waits the compiler derives for the prefetched loads count the instructions issued after them
// instead of also waiting for the acknowledgement of the band's last stores and atomics (the counter is decremented
// in order, and with a store on only some paths the wait has to assume it was not issued).
//
// CHB > 1: the block holds CHB channels of one (batch, group) pair, each with its own waves.  The channels' dB / dC
// contributions of a band meet in LDS and leave as one atomic per element and block: the atomics are performed at
// the memory side, line by line, and cost the kernel a third to a half of its time when every channel issues its own.
//
// PK > 1 (with CHB > 1): narrow planes packed PK to a wave as in the forward (wave_pack() in snd_device.h); the block
// then holds CHB * PK channels, and the planes of a wave are added up with the waves of the block.
//
// XW: the most waves a block may have, 8 or (two channels of five to eight segments) 16.
//
// EXT: the launch works on one column group of a wide plane (wave_wide() in snd_device.h), segments seg0 .. seg0+nseg-1;
// the groups are launched right to left.  The group's last wave takes G, Gs, a of the column on its right from global
// memory (with the band's loads, three values per state and row spread over the lanes of one register), where the
// first wave of the group on the right left them, and puts them into the LDS slot a neighbouring wave would have filled.
//
// SPL (with EXT): a split plane (wave_bwd_split() in snd_device.h): the block works on one half of the segments of two
// channels, the two halves of a channel pair are blocks of the same launch, and the hand-over goes through tagged
// words that the left half's edge wave checks.
template <typename T, int NS, int CPL, bool VEC, bool DO32, bool EVEN, int CHB, int PK, int XW, bool EXT = false, bool SPL = false>
__global__ __launch_bounds__(64 * (XW + (SPL ? 1 : 0))) void wave_bwd_kernel(const snd_bwd_params p, const WaveGeo wg) {
    constexpr int R = wave_band_rows(NS);            // rows per band
    static_assert(!EXT || (CHB == (SPL ? 2 : 1) && PK == 1 && CPL == 1 && (!EVEN || SPL)), "column groups: one channel per block, one column per lane");
    static_assert(!SPL || EXT, "a split plane hands over like a column group");
    static_assert(CHB == 1 || CPL == 1, "shared atomics: one column per lane");
    static_assert(PK == 1 || (CHB > 1 && !EVEN), "packed planes share their atomics");
    constexpr int S = 64 / PK;                       // lanes per plane
    constexpr int kItems = R * NS * 2;               // dB and dC rows of a band
    static_assert(kItems % CHB == 0, "the waves of a segment take equal shares of a band's dB / dC rows");
    static_assert(XW == kMaxSeg || (CHB == 2 && NS <= 2 && PK == 1), "blocks of 16 waves: two channels, one or two states");
    // Two buffers, so that one barrier per band is enough - where they leave the CU its blocks: with three states they
    // would be 48 KB, two blocks per CU instead of four (32x12288x7x7: 0.50 ms against 0.31 with one buffer).
    constexpr int kXBuf = CHB == 1 ? 1 : (NS >= 3 || XW > 8) ? 1 : 2;
    constexpr int kXWaves = CHB == 1 ? 1 : XW;
    __shared__ float sX[kXBuf][kXWaves][CHB == 1 ? 1 : kItems][CHB == 1 ? 1 : 64];
    // load a band's inputs one band ahead (with three or four states it measured 20 % slower, and with two columns per
    // lane the registers are needed elsewhere)
    constexpr bool PF = NS <= 2 && CPL == 1;
    // what a wave leaves for the wave on its left: {G, Gs, a, -} at its first column, per band parity, row and
    // state.  Wave w writes slot w and reads slot w+1; the slot after the last wave stays zero.
    __shared__ float4 sHO[2][CHB][kMaxSeg + 1][R][NS];

    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = wg.rg, rd = wg.rd;
    const int nseg = wg.nseg;
    const int lane = threadIdx.x & 63, wi = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int kc = CHB > 1 ? wi / nseg : 0, w = PK > 1 ? 0 : wi - kc * nseg;     // channel of the block, segment of the channel
    const int sl = PK > 1 ? lane % S : lane;         // the lane inside its plane
    int pair, chunk, half = 0;
    if (SPL) {
        // Blocks are dealt to the XCDs in turn (block i to XCD i % 8); the two halves of a channel pair take consecutive
        // places of one XCD, the right half - which never waits - first: what it hands over then passes through the L2
        // the left half reads from.
        const int id = blockIdx.x, slot = id >> 3, unit = (slot >> 1) * 8 + (id & 7), nCP = (rg + 1) >> 1;
        half = slot & 1;
        if (unit >= sh.batch * G * nCP) return;
        pair = unit / nCP;
        chunk = unit - pair * nCP;
    } else if (!wave_job2(wg, sh.batch * G, pair, chunk)) {
        return;
    }
    if (SPL && wi == CHB * nseg) {
        // The block's extra wave.  In a left half it fetches what the right half has left for the coming band - the tagged
        // words of both channels, one word per lane, loaded again until every tag is the band's (a bounded number of
        // times) - and puts the values where a wave on the right of the half's last segment would have put them, one
        // step ahead of the wave that reads them.  Loads that pass the L2 by take several microseconds behind the
        // kernel's dB / dC atomics, and a wave's memory instructions complete in order: issued by the half's last wave
        // itself, one such load per band held up its whole queue (0.46 instead of 0.36 ms at 256 planes of 512x512).
        // This wave has no other loads.  It joins every barrier of the block; in a right half that is all it does.
        constexpr int kWords = 3 * NS * R;           // (at most 12)
        const int hk = lane >> 4, hl = lane & 15, hq = hl / (NS * R), hn = (hl / R) % NS, hr = hl % R;
        int b_, g_;
        wave_pair_split(wg, pair, G, b_, g_);
        const int64_t plane = ((int64_t)b_ * Dm + g_ * rg + min(chunk * CHB + hk, rg - 1)) * N + hn;
        const bool fetch = half == 1 && hk < CHB && hl < kWords;
        const uint64_t *src = (const uint64_t *)(wg.bcol + (fetch ? plane : 0) * wave_split_words(wg) + 2 * (hq * R + hr));
        bool dead = false;
        lds_barrier();                               // the zeroed slots
        for (int s = 0; s < wg.nBands + nseg; ++s) {
            if (half == 1 && s < wg.nBands) {
                const int band = wg.nBands - 1 - s;
                const bool mine = fetch && band * R + hr < H;   // (rows past the plane's last are never swept: no words for them)
                const uint32_t want = (uint32_t)band + 1u;
                uint64_t word = 0;
                for (int polls = 0;; ++polls) {
                    if (mine) word = __hip_atomic_load(src + (int64_t)band * (3 * R), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (dead || __builtin_amdgcn_ballot_w64(mine && (uint32_t)(word >> 32) != want) == 0) break;
                    if (polls >= wg.spinLimit) {
                        dead = true;
                        __hip_atomic_store(wg.sync + kErrorWord, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(SND_POLL_SLEEP);
                }
                if (fetch) ((float *)&sHO[(s + 1) & 1][hk < CHB ? hk : 0][nseg][hr][hn])[hq] = dead ? __builtin_nanf("") : __builtin_bit_cast(float, (uint32_t)word);   // (never plausible numbers)
            }
            lds_barrier();
        }
        return;
    }
    const int sg = EXT ? (SPL ? (half ? 0 : wg.seg0) : wg.seg0) + w : w;   // this wave's segment of the plane
    chunk = (chunk * CHB + kc) * PK + (PK > 1 ? lane / S : 0);       // (packed: a lane's own from here on)
    // A wave (a plane of a wave) past the last channel of its group repeats that channel (identical du / ddelta
    // stores) and adds nothing.
    const bool active = CHB == 1 || chunk < rg;
    chunk = min(chunk, rg - 1);
    int b, g;
    wave_pair_split(wg, pair, G, b, g);
    const int c = g * rg + chunk, cd = rd == 1 ? c : c / rd;   // channel of u, of delta
    // channel offsets: in the scalar base pointers, or (packed) in the lanes' offsets
    const int cB = PK > 1 ? 0 : c, chB = PK > 1 ? 0 : chunk, cL = PK > 1 ? c : 0, chL = PK > 1 ? chunk : 0;
    const bool multi = nseg > 1;
    if (threadIdx.x < 2 * R * NS)
#pragma unroll
        for (int q = 0; q < CHB; ++q) sHO[threadIdx.x / (R * NS)][q][nseg][threadIdx.x % (R * NS) / NS][threadIdx.x % NS] = make_float4(0.f, 0.f, 0.f, 0.f);

    const bool fv = f.directions == SND_DIR_CORNERS && (g & 2), fh = f.directions == SND_DIR_CORNERS && (g & 1);
    const int r0m = fv ? H - 1 : 0, rs = fv ? -1 : 1;
    // Mirrored order: this lane owns scan columns jm0 .. jm0+CPL-1 and walks them downwards (its local index t is
    // scan column jm0 + CPL-1-t); in natural order (row checkpoints, recomputation) lane l owns columns jn0 ...
    const bool bar = PK == 8 && sl == 0;             // (eight planes per wave) the plane's barrier lane: mirrored column 7
    const int jm0 = PK > 1 ? S - 1 - sl : (sg * kSeg + 63 - lane) * CPL;
    const bool jin = EVEN || jm0 < W;
    const int jc = jin ? jm0 : W - CPL;
    const int mc = fh ? W - CPL - jc : jc;           // memory column of the lane's lowest address
    const int jn0 = PK == 8 ? max(sl - 1, 0) : (sg * kSeg + sl) * CPL;
    // the mirror lane inside the plane (eight planes: lanes 1..7 among themselves, the barrier lane stays)
    const int rev_addr = PK == 8 ? ((lane - sl) + (sl == 0 ? 0 : 8 - sl)) * 4 : PK > 1 ? ((lane - sl) + S - 1 - sl) * 4 : (63 - lane) * 4;
    auto mirror = [&](float v) {
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(rev_addr, __builtin_bit_cast(int, v)));
    };
    auto bcast = [](float v, int src_lane) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src_lane));
    };

    float Av[NS], A2[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        Av[n] = f.A[(int64_t)c * f.A_d_stride + (int64_t)n * f.A_dstate_stride];   // (NS == N)
        A2[n] = Av[n] * kLog2e;
    }
    const float ld = f.A_decay ? __log2f(f.A_decay[0]) : 0.f;
    const float Dv = f.D ? f.D[c] : 0.f;
    const float bias = f.delta_bias ? f.delta_bias[cd] : 0.f;
    const bool softplus = f.delta_softplus != 0;
    const bool want_decay = p.dA_decay != nullptr;

    constexpr int ESZ = (int)sizeof(T);
    using DoT = typename std::conditional<DO32, float, T>::type;
    constexpr int DSZ = (int)sizeof(DoT);
    const T *Bb = (const T *)f.B + (int64_t)b * f.B_batch_stride + (int64_t)g * f.B_group_stride;
    const T *Cb = (const T *)f.C + (int64_t)b * f.C_batch_stride + (int64_t)g * f.C_group_stride;
    const T *ub = (const T *)f.u + (int64_t)b * f.u_batch_stride + (int64_t)(f.u_shared ? chB : cB) * f.u_d_stride;
    const T *db = (const T *)f.delta + (int64_t)b * f.delta_batch_stride + (int64_t)(PK > 1 ? 0 : cd) * f.delta_d_stride;
    // fused CrossMerge: dout is the gradient of the merged output, shared by the groups and scaled by the channel's weight
    const bool merge = f.merge != 0;
    // (times NaN if the saved state was written by the other kernel family: see kTagWave)
    const float wm = (merge && f.merge_weights ? f.merge_weights[c] : 1.f) * tag_poison(wg.tag, kTagWave);
    const DoT *dob = (const DoT *)p.dout + (int64_t)b * p.dout_batch_stride + (int64_t)(merge ? chB : cB) * p.dout_d_stride;
    T *dub = (T *)p.du + ((int64_t)b * Dm + cB) * H * W;                // du, ddelta: dense [b, c, H, W]
    T *ddb = (T *)p.ddelta + ((int64_t)b * Dm + cB) * H * W;
    float *dBg = p.dB + ((int64_t)b * G + g) * N * H * W;               // dense [b, g, N, H, W]
    float *dCg = p.dC + ((int64_t)b * G + g) * N * H * W;
    // (stores and atomics go through buffer descriptors: lanes and rows outside the plane are dropped by the hardware's
    // range check instead of a branch, see buf_rsrc() in snd_device.h)
    const __amdgpu_buffer_rsrc_t rdu = buf_rsrc(dub), rdd = buf_rsrc(ddb), rdB = buf_rsrc(dBg), rdC = buf_rsrc(dCg);
    // byte steps from one scan row to the next (negative when the group scans bottom-up) and column offsets
    const int UhB = (int)f.u_h_stride * ESZ * rs, DhB = (int)f.delta_h_stride * ESZ * rs, BhB = (int)f.B_h_stride * ESZ * rs,
              ChB = (int)f.C_h_stride * ESZ * rs, DohB = (int)p.dout_h_stride * DSZ * rs, WB = W * ESZ * rs, W4 = W * 4 * rs;
    const int64_t BsB = f.B_dstate_stride * ESZ, CsB = f.C_dstate_stride * ESZ, HW4 = (int64_t)H * W * 4;
    const uint32_t colB = (uint32_t)mc * ESZ, col4 = (uint32_t)mc * 4;
    const uint32_t colU = colB + (uint32_t)(f.u_shared ? chL : cL) * (uint32_t)f.u_d_stride * ESZ,
                   colD = colB + (uint32_t)(PK > 1 ? cd : 0) * (uint32_t)f.delta_d_stride * ESZ,
                   colO = (uint32_t)mc * DSZ + (uint32_t)(merge ? chL : cL) * (uint32_t)p.dout_d_stride * DSZ,
                   colG = colB + (uint32_t)cL * (uint32_t)(H * W) * ESZ;                  // du, ddelta

    // saved state of this plane set (layouts in snd_device.h)
    const int64_t plane0 = ((int64_t)b * Dm + c) * N;
    const float *xv = f.x_v + plane0 * wave_xv_plane(wg) + jn0;
    const float *xh = f.x + plane0 * wave_x_plane(wg) + (int64_t)sg * 2 * wg.Hp;
    const float *xs = f.x_sd + plane0 * wave_x_plane(wg) + (int64_t)sg * 2 * wg.Hp;
    // (column groups) lane (q*NS + n)*R + r fetches G (q = 0), Gs (1), a (2) of the group on the right: row r of a band, state n
    constexpr int kExtLanes = 3 * NS * R;
    const int el = lane < kExtLanes ? lane : 0, eq = el / (NS * R), er = el % R, gq = EXT ? wg.seg0 / kMaxSeg : 0;
    const float *ebase = EXT ? wg.bcol + (plane0 + (el / R) % NS) * wave_bcol_plane(wg)
                               + (int64_t)min(gq + 1, wave_groups(wg.nsegAll) - 1) * 3 * wg.Hp + eq * wg.Hp : nullptr;
    float *eout = EXT ? wg.bcol + plane0 * wave_bcol_plane(wg) + (int64_t)gq * 3 * wg.Hp : nullptr;
    const bool ext_in = EXT && (SPL ? half == 1 : wg.extR != 0) && w == nseg - 1 && !(SND_WAVE_ABLATE & 512),
               ext_out = EXT && (SPL ? half == 0 : wg.extL != 0) && w == 0 && !(SND_WAVE_ABLATE & 256);
    // (split planes) the tagged words of the plane's first state
    float *eouttag = SPL ? wg.bcol + plane0 * wave_split_words(wg) : nullptr;

    // Inputs of one band.  Rows wait as raw bits in mirrored lane order; lanes beyond the last column read the
    // last columns (always in bounds) and only their dout is masked to zero where it is used, which makes every
    // adjoint there exactly zero.  h0: h of the row above the band in natural order; dtop: that row's delta (its a is
    // recomputed).  ch, cs, ca: what entered
    // the segment from the left on rows i0-1 .. i0+R-1, one row per lane.
    typedef WaveRaw<T, CPL, VEC> Raw;
    typedef WaveRaw<DoT, CPL, VEC> RawO;
    struct In { Raw u[R], d[R], b[R][NS], c[R][NS]; RawO o[R]; Raw dtop; float h0[NS][CPL], ch[NS], cs[NS], ca[NS], e; };
    // Every band issues the same loads on every path (the wait counters the compiler derives for the prefetch
    // need that): rows past the end of a ragged last band read the last row again and are never used.
    auto load_band = [&](In &q, int band) {
        const int i0 = band * R;
        const int m0 = mad24(i0, rs, r0m);           // memory row of the band's first scan row
        uint32_t ou = mad24(m0, UhB * rs, colU), od = mad24(m0, DhB * rs, colD), oo = mad24(m0, DohB * rs, colO),
                 ob = mad24(m0, BhB * rs, colB), oc = mad24(m0, ChB * rs, colB);
        wave_ld(q.dtop, db, band > 0 ? od - DhB : od);   // (the first band has no row above: any row, never used)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            wave_ld(q.u[r], ub, ou);
            wave_ld(q.d[r], db, od);
            wave_ld(q.o[r], dob, oo);
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                const int sn = n;
                wave_ld(q.b[r][n], (const T *)((const char *)Bb + sn * BsB), ob);
                wave_ld(q.c[r][n], (const T *)((const char *)Cb + sn * CsB), oc);
            }
            const bool more = i0 + r + 1 < H;
            ou += more ? UhB : 0; od += more ? DhB : 0; oo += more ? DohB : 0; ob += more ? BhB : 0; oc += more ? ChB : 0;
        }
        const int row = i0 - 1 + lane;
#pragma unroll
        for (int n = 0; n < NS; ++n) {
            q.ch[n] = 0.f; q.cs[n] = 0.f; q.ca[n] = 0.f;
#pragma unroll
            for (int k = 0; k < CPL; ++k) q.h0[n][k] = 0.f;
            {
                if (band > 0) {
                    const float *src = xv + (int64_t)n * wave_xv_plane(wg) + (int64_t)(band - 1) * wg.Wp;
                    if (CPL == 2) {
                        const wave_f2 v = __builtin_nontemporal_load((const wave_f2 *)src);
                        q.h0[n][0] = v.x; q.h0[n][CPL - 1] = v.y;
                    } else {
                        q.h0[n][0] = __builtin_nontemporal_load(src);
                    }
#pragma unroll
                    for (int k = 0; k < CPL; ++k)
                        if (PK == 8) q.h0[n][k] = bar ? 0.f : q.h0[n][k];
                }
                if (sg > 0 && lane <= R && row >= 0) {
                    const int64_t o = (int64_t)n * wave_x_plane(wg) + row;
                    q.ch[n] = xh[o];
                    q.ca[n] = xh[o + wg.Hp];
                    q.cs[n] = xs[o];
                }
            }
        }
        if (EXT && !SPL) q.e = ebase[i0 + er];       // (by every wave, like the other loads; only the group's last wave uses it)
        // (split planes: by the left half's edge wave alone - the load passes the L2 by, takes that much longer, and every
        // load behind it in a wave's queue waits for it: issued by all waves it cost 256 planes of 512x512 0.07 of 0.44 ms)
    };
    // the lane's CPL values in its walking order t (element e of the raw bits is t = CPL-1-e, or t = e when fh)
    auto unpack = [&](const auto &q, float (&v)[CPL]) {
#pragma unroll
        for (int k = 0; k < CPL; ++k) v[k] = wave_elem(q, k);
        if (CPL == 2 && !fh) { const float t = v[0]; v[0] = v[CPL - 1]; v[CPL - 1] = t; }
    };

    float Gd[NS][CPL], ad[NS][CPL], GdEdge[NS];     // G, a of the row below at this lane's columns; G[i+1, S*(w+1)]
    float dA_acc[NS];
    float dec_acc = 0.f, dD_acc = 0.f, dbias_acc = 0.f, dw_acc = 0.f;
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        GdEdge[n] = 0.f; dA_acc[n] = 0.f;
#pragma unroll
        for (int k = 0; k < CPL; ++k) { Gd[n][k] = 0.f; ad[n][k] = 0.f; }
    }
    int step = nseg - 1 - w;                         // the waves on the right go first
    const bool hands_over = multi && w > 0;

    // one band from `cur`, with the loads of the band above issued into `nxt` first
    auto do_band = [&](In &cur, In &nxt, int band) {
        if (!PF) load_band(cur, band);
        const int i0 = band * R;
        // (the recomputation at a raised wave priority, the sweep with its stores and atomics at the default one: the
        // waves sharing a SIMD then interleave the two phases.  2 x 192 x 200x336, two states: 0.419 -> 0.400 ms, four
        // states at 56x56 0.662 -> 0.647, the one-state workloads unchanged)
        __builtin_amdgcn_s_setprio(3);

        // ---- recompute h, s on the band's rows (with the columns); results back in mirrored order.
        // Index t of the mirrored order is natural column index CPL-1-t of the lane that holds the same columns.
        float hT[R][NS][CPL], sT[R][NS][CPL], aT[R][NS][CPL], dl[R][CPL], dsp[R][CPL], uu[R][CPL], hTop[NS][CPL];
        {
            float hp[NS][CPL], ap[NS][CPL], hdiag[NS];
            // a of the row above the band, from that row's delta (zero above the first band, and in a barrier lane)
            float dtop[CPL];
            unpack(cur.dtop, dtop);
#pragma unroll
            for (int t = 0; t < CPL; ++t) {
                const float raw = dtop[t] + bias;
                float sg;
                dtop[t] = softplus ? softplus20(raw, sg) : raw;
            }
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                hdiag[n] = bcast(cur.ch[n], 0);
#pragma unroll
                for (int k = 0; k < CPL; ++k) {
                    hp[n][k] = cur.h0[n][k];
                    const float at = band > 0 ? fast_exp2(fmaf(dtop[CPL - 1 - k], A2[n], ld)) : 0.f;
                    ap[n][k] = mirror(at);
                    if (PK == 8) ap[n][k] = bar ? 0.f : ap[n][k];
                    hTop[n][CPL - 1 - k] = mirror(cur.h0[n][k]);
                }
            }
            // What the rows need that does not depend on the rows above them - softplus, delta' * u, and their
            // copies in natural lane order - for the whole band at once: R independent chains of transcendentals and
            // a train of lane reversals in flight, instead of one chain and three round trips in front of every row's scan.
            float dln_[R][CPL], dlun_[R][CPL], bn_[R][NS][CPL];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                unpack(cur.u[r], uu[r]);
                unpack(cur.d[r], dl[r]);
#pragma unroll
                for (int t = 0; t < CPL; ++t) {
                    const float raw = dl[r][t] + bias;
                    float sg = 1.f;
                    dl[r][t] = softplus ? softplus20(raw, sg) : raw;
                    dsp[r][t] = sg;
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int t = 0; t < CPL; ++t) {
                    dln_[r][CPL - 1 - t] = mirror(dl[r][t]);
                    dlun_[r][CPL - 1 - t] = mirror(dl[r][t] * uu[r][t]);
                }
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    float bm[CPL];
                    unpack(cur.b[r][n], bm);
#pragma unroll
                    for (int t = 0; t < CPL; ++t) bn_[r][n][CPL - 1 - t] = mirror(bm[t]);
                }
            }
            // (every row of the band, also those past the plane's last row in a ragged last band: they read the last row's
            // inputs again, their dout is taken as zero below, and nothing of them is stored)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                {
                    const float (&dln)[CPL] = dln_[r], (&dlun)[CPL] = dlun_[r];
#pragma unroll
                    for (int n = 0; n < NS; ++n) {
                        // (rows past the plane's last have no column checkpoint: zeros, so that what is computed there is finite)
                        const bool rin = EVEN || i0 + r < H;
                        const float hin = rin ? bcast(cur.ch[n], r + 1) : 0.f, sin_ = rin ? bcast(cur.cs[n], r + 1) : 0.f, ain = rin ? bcast(cur.ca[n], r + 1) : 0.f;
                        float a[CPL], bu[CPL], y[CPL], h[CPL], s[CPL];
#pragma unroll
                        for (int k = 0; k < CPL; ++k) {
                            a[k] = fast_exp2(fmaf(dln[k], A2[n], ld));
                            bu[k] = bn_[r][n][k] * dlun[k];
                            if (PK == 8) { a[k] = bar ? 0.f : a[k]; bu[k] = bar ? 0.f : bu[k]; }   // the barrier lane's map is (0, 0)
                        }
                        const float a_l = from_prev_lane_pk<PK>(a[CPL - 1], ain, sl == 0);                 // a[i, j-1] of the lane's first column
                        const float h_d = from_prev_lane_pk<PK>(hp[n][CPL - 1], hdiag[n], sl == 0);        // h[i-1, j-1]
#pragma unroll
                        for (int k = 0; k < CPL; ++k) {
                            const float al = k == 0 ? a_l : a[k > 0 ? k - 1 : 0], hd = k == 0 ? h_d : hp[n][k > 0 ? k - 1 : 0];
                            const float X = fmaf(-0.5f * (ap[n][k] + al), hd, hp[n][k]);
                            y[k] = fmaf(a[k], X, bu[k]);
                        }
                        wave_row_solve<CPL, PK>(a, y, bu, hin, sin_, h, s);
#pragma unroll
                        for (int k = 0; k < CPL; ++k) {
                            hT[r][n][CPL - 1 - k] = mirror(h[k]);
                            sT[r][n][CPL - 1 - k] = mirror(s[k]);
                            aT[r][n][CPL - 1 - k] = mirror(a[k]);
                            hp[n][k] = h[k];
                            ap[n][k] = a[k];
                        }
                        hdiag[n] = hin;
                    }
                }
            }
        }

        // The loads of the band above are issued here, between the two phases, not at the top of the band: a wave
        // can have 63 memory instructions in flight, and at the top of a band the 2 stores and 2N atomics per row of
        // the sweep just finished still are (40 loads on top of them stalled the issue for a quarter of the kernel);
        // here they have had the whole recomputation to complete.  Unconditionally (band 0 once more): a skipped
        // load would leave two paths with different numbers of loads in flight, and the waits follow the smaller.
        if (PF) load_band(nxt, max(band - 1, 0));
        __builtin_amdgcn_s_setprio(0);

        // ---- adjoint sweep over the band's rows, bottom-up (against the columns: local index t walks downwards)
        // (column groups) what the group on the right left for this band goes where a wave on the right would have put
        // it: the group's last wave fills its own neighbour slot, one word per lane, and the rows below read it as ever
        if (EXT && !SPL && ext_in && lane < kExtLanes) ((float *)&sHO[(step + 1) & 1][kc][nseg][er][(el / R) % NS])[eq] = cur.e;
        // (from the band's last row up, rows past the plane's last included: their offsets are never used)
        const int mlast = mad24(i0 + R - 1, rs, r0m);
        uint32_t og = mad24(mlast, WB * rs, colG), o4 = mad24(mlast, W4 * rs, col4);   // du / ddelta and dB / dC offsets of the row
#pragma unroll
        for (int r = R - 1; r >= 0; --r) {
            {
                // whether this lane's cells of the row are inside the plane: outside, dout counts as zero - which makes
                // every adjoint there exactly zero - and nothing is stored or added
                const bool in_plane = jin && (EVEN || i0 + r < H);
                float dov[CPL], dlu[CPL], qsum[CPL], psum[CPL];
                unpack(cur.o[r], dov);
#pragma unroll
                for (int t = 0; t < CPL; ++t) {
                    dov[t] = in_plane ? wm * dov[t] : 0.f;
                    dlu[t] = dl[r][t] * uu[r][t];
                    qsum[t] = 0.f;
                    psum[t] = 0.f;
                }
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    // what the segment on the right left for this row: G, Gs, a at column S*(w+1)
                    const float4 in = (PK > 1 && NS <= 2) ? make_float4(0.f, 0.f, 0.f, 0.f) : sHO[(step + 1) & 1][kc][w + 1][r][n];   // (packed planes have no neighbour)
                    const float hin = (EVEN || i0 + r < H) ? bcast(cur.ch[n], r + 1) : 0.f;   // h[i, S*w-1]
                    float Bv[CPL], Cv[CPL], a[CPL], bu[CPL], dyC[CPL], z[CPL], ya[CPL], ys[CPL], Gt[CPL], Gst[CPL];
                    unpack(cur.b[r][n], Bv);
                    unpack(cur.c[r][n], Cv);
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        a[t] = aT[r][n][t];
                        bu[t] = Bv[t] * dlu[t];
                        dyC[t] = dov[t] * Cv[t];
                    }
                    const float a_r0 = from_prev_lane_pk<PK>(a[CPL - 1], in.z, sl == 0);               // a[i, j+1] of the lane's first column
                    const float Gdg0 = from_prev_lane_pk<PK>(Gd[n][CPL - 1], GdEdge[n], sl == 0);      // G[i+1, j+1]
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        const float ar = t == 0 ? a_r0 : a[t > 0 ? t - 1 : 0], gdg = t == 0 ? Gdg0 : Gd[n][t > 0 ? t - 1 : 0];
                        z[t] = fmaf(-0.5f * (ar + ad[n][t]), gdg, dyC[t] + Gd[n][t]);
                        ya[t] = a[t] * z[t];
                        ys[t] = -a[t] * dyC[t];
                    }
                    wave_row_solve<CPL, PK>(a, ya, ys, in.x, in.y, Gt, Gst);           // G[i,j], Gs[i,j]
                    const float Gr0 = from_prev_lane_pk<PK>(Gt[CPL - 1], in.x, sl == 0), Gsr0 = from_prev_lane_pk<PK>(Gst[CPL - 1], in.y, sl == 0);
                    const float hl_last = from_next_lane_pk<PK>(hT[r][n][0], hin, sl == S - 1);   // h[i, j-1] of the lane's last column
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        const float Gr = t == 0 ? Gr0 : Gt[t > 0 ? t - 1 : 0], Gsr = t == 0 ? Gsr0 : Gst[t > 0 ? t - 1 : 0];
                        float g_ = Gr + z[t], gs = Gsr - dyC[t];
                        if (PK == 8) { g_ = bar ? 0.f : g_; gs = bar ? 0.f : gs; }         // (what the barrier lane fetched is another plane's)
                        const float dbu = fmaf(0.25f, dyC[t], g_ + gs);
                        const float hv = hT[r][n][t], sv = sT[r][n][t];
                        const float h_l = t == CPL - 1 ? hl_last : hT[r][n][t < CPL - 1 ? t + 1 : 0];
                        const float h_u = r > 0 ? hT[r > 0 ? r - 1 : 0][n][t] : hTop[n][t];
                        const float hs = hv - sv, sb = sv - bu[t];
                        const float cross = fmaf(Gd[n][t], h_l, Gr * h_u);
                        const float da = fmaf(-0.5f * a[t], cross, fmaf(g_, hs, (g_ + gs) * sb));
                        dA_acc[n] = fmaf(dl[r][t], da, dA_acc[n]);
                        if (want_decay) dec_acc += da;
                        qsum[t] = fmaf(dbu, Bv[t], qsum[t]);
                        psum[t] = fmaf(Av[n], da, psum[t]);
                        ya[t] = dbu * dlu[t];                                          // dB, dC contributions (reusing the arrays)
                        ys[t] = dov[t] * fmaf(0.25f, bu[t], hs);
                    }
                    if (CHB > 1) {
                        sX[kXBuf == 2 ? step & 1 : 0][wi][(r * NS + n) * 2][lane] = active ? ya[0] : 0.f;
                        sX[kXBuf == 2 ? step & 1 : 0][wi][(r * NS + n) * 2 + 1][lane] = active ? ys[0] : 0.f;
                    } else if (!(SND_WAVE_ABLATE & 64) || ya[0] == 1234.5f) {
#pragma unroll
                        for (int e = 0; e < CPL; ++e) {                                // memory order
                            const int t = fh ? e : CPL - 1 - e;
                            const float vb = (CPL == 2 && t == 1) ? ya[CPL - 1] : ya[0], vc = (CPL == 2 && t == 1) ? ys[CPL - 1] : ys[0];
                            const uint32_t off = in_plane ? o4 + 4u * e : kBufOOB;
                            buf_add_f32(rdB, off, (uint32_t)(n * HW4), vb);
                            buf_add_f32(rdC, off, (uint32_t)(n * HW4), vc);
                        }
                    }
                    GdEdge[n] = in.x;
#pragma unroll
                    for (int t = 0; t < CPL; ++t) { Gd[n][t] = Gt[t]; ad[n][t] = a[t]; }
                    if (hands_over && lane == 63) sHO[step & 1][kc][w][r][n] = make_float4(Gt[CPL - 1], Gst[CPL - 1], a[CPL - 1], 0.f);
                    if (EXT && !SPL && ext_out && lane == 63) {   // for the column group on the left
                        float *d = eout + (int64_t)n * wave_bcol_plane(wg) + i0 + r;
                        d[0] = Gt[CPL - 1];
                        d[wg.Hp] = Gst[CPL - 1];
                        d[2 * wg.Hp] = a[CPL - 1];
                    }
                    if (SPL && ext_out && lane == 63) {           // for the left half: tagged with the band
                        float *d = eouttag + (int64_t)n * wave_split_words(wg) + (int64_t)band * (6 * R) + 2 * r;
                        const float tg = __builtin_bit_cast(float, (uint32_t)band + 1u);
                        st2_coherent(d, Gt[CPL - 1], tg);
                        st2_coherent(d + 2 * R, Gst[CPL - 1], tg);
                        st2_coherent(d + 4 * R, a[CPL - 1], tg);
                    }
                }
                {
                    float duv[CPL], ddl[CPL];
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        duv[t] = fmaf(Dv, dov[t], dl[r][t] * qsum[t]);
                        ddl[t] = fmaf(uu[r][t], qsum[t], psum[t]) * dsp[r][t];
                        dD_acc = fmaf(dov[t], uu[r][t], dD_acc);
                        dw_acc = fmaf(duv[t], uu[r][t], dw_acc);
                        dbias_acc += ddl[t];
                    }
                    if (CPL == 2 && !fh) {                                             // to memory order
                        float t_ = duv[0]; duv[0] = duv[CPL - 1]; duv[CPL - 1] = t_;
                        t_ = ddl[0]; ddl[0] = ddl[CPL - 1]; ddl[CPL - 1] = t_;
                    }
                    if (!(SND_WAVE_ABLATE & 128) || duv[0] == 1234.5f) {
                        wave_st_buf<T, CPL, VEC>(rdu, in_plane ? og : kBufOOB, duv);
                        wave_st_buf<T, CPL, VEC>(rdd, in_plane ? og : kBufOOB, ddl);
                    }
                }
                og -= WB;
                o4 -= W4;
            }
        }
        if (CHB > 1) {
            // Wave kc of a segment adds up rows kc, kc + CHB, ... of what the segment's CHB waves left and issues
            // their atomics.
            lds_barrier();
            if (!(SND_WAVE_ABLATE & 64))
#pragma unroll
            for (int m = 0; m < kItems / CHB; ++m) {
                const int it = m * CHB + kc, r = it / (2 * NS), n = (it >> 1) % NS;
                float v = 0.f;
#pragma unroll
                for (int q = 0; q < CHB; ++q)
#pragma unroll
                    for (int k = 0; k < PK; ++k) v += sX[kXBuf == 2 ? step & 1 : 0][w + q * nseg][it][PK > 1 ? sl + k * S : lane];
                const uint32_t off = mad24(mad24(i0 + r, rs, r0m), W * 4, (int)col4);
                const bool in_plane = jin && (PK == 1 || lane < S) && (EVEN || i0 + r < H);
                buf_add_f32(buf_rsrc((it & 1) ? dCg : dBg), in_plane ? off : kBufOOB, (uint32_t)(n * HW4), v);
            }
            if (kXBuf == 1) lds_barrier();
            ++step;
        } else if (multi) { lds_barrier(); ++step; }
    };

    In sA;
    if (PF) load_band(sA, wg.nBands - 1);
    // (nothing in flight on the way into the band loop: its first waits then follow the loop's own path as well)
    if (PF) __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    lds_barrier();                                   // the zeroed slot
    if (SPL) lds_barrier();                          // (and what the block's extra wave has fetched for the first band)
    if (multi)
        for (int e = 0; e < (nseg - 1 - w) * (CHB > 1 && kXBuf == 1 ? 2 : 1); ++e) lds_barrier();
    if (PF) {
        In sB;
        for (int band = wg.nBands - 1; band >= 0; band -= 2) {
            do_band(sA, sB, band);
            if (band > 0) do_band(sB, sA, band - 1);
        }
    } else {
        for (int band = wg.nBands - 1; band >= 0; --band) do_band(sA, sA, band);
    }
    if (multi)
        for (int e = 0; e < w * (CHB > 1 && kXBuf == 1 ? 2 : 1); ++e) lds_barrier();

    // ---- per-channel sums leave the kernel: one atomic per wave and value
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        const float t = wave_sum_to_plane_last<PK>(dA_acc[n]);
        if (sl == S - 1 && n < N && active) wave_glb_add(p.dA + (int64_t)c * N + n, t);
    }
    {
        const float td = wave_sum_to_plane_last<PK>(dD_acc), tb = wave_sum_to_plane_last<PK>(dbias_acc);
        if (sl == S - 1 && active) {
            if (p.dD) wave_glb_add(p.dD + c, td);
            if (p.ddelta_bias) wave_glb_add(p.ddelta_bias + c, tb);
        }
        // Fused CrossMerge: weight * d(weight) = <weighted dout, result of the channel>, and since the result is
        // linear in u (D*u plus a recurrence linear in B*delta'*u) that inner product equals <du, u>.
        if (merge && p.dmerge) {
            const float tw = wave_sum_to_plane_last<PK>(dw_acc);
            if (sl == S - 1 && active) wave_glb_add(p.dmerge + c, tw);
        }
    }
    if (want_decay) {
        const float t = wave_sum_to_plane_last<PK>(dec_acc);
        if (sl == S - 1 && active) wave_glb_add(p.dA_decay, t / f.A_decay[0]);
    }
}

static inline bool wave_aligned_b(const void *ptr, int64_t esz, int bytes, std::initializer_list<int64_t> strides) {
    if ((uintptr_t)ptr % bytes) return false;
    for (int64_t st : strides)
        if ((st * esz) % bytes) return false;
    return true;
}

// Channels per block.  Sharing the atomics needs the channels' waves in one block, and a block may hold
// kWaveShareWaves of them; small launches spread further with one channel per block.  Measured: four one-wave
// channels pay from 512 planes on (56x56); with a full load of waves, one or two states, four channels of two segments
// (64x96x112x112, two states: 0.85 -> 0.78 ms over two channels) and two channels of three or four segments
// (4x256x256x256, one state: 0.50 -> 0.33 ms, two states 0.99 -> 0.59; 16x96x160x160: 0.36 -> 0.32); with three or
// four states two channels of two segments, and no more (blocks of 6 or 8 waves lost 14 to 50 %).  Planes of five to
// eight segments, one or two states: two channels in a block of 10 to 16 waves once there are more planes than CUs
// (2x256x512x512, one state: 1.00 -> 0.67 ms; 4x192x300x300: 0.75 -> 0.71; with 256 planes the blocks would fill half
// the CUs: 0.46 -> 0.62).
static inline int wave_bwd_share(const snd_shape &sh, const WaveGeo &wg) {
    const int64_t waves = (int64_t)sh.batch * sh.dim * wg.nseg;
    if (wg.cpl != 1) return 1;
    if (wg.nseg == 1) return waves >= 512 ? 4 : 1;
    if (waves < 2048) return 1;
    if (sh.dstate > 2) return wg.nseg == 2 ? 2 : 1;
    if (wg.nseg > 4) return (int64_t)sh.batch * sh.dim > 256 ? 2 : 1;       // blocks of 10 to 16 waves
    return wg.nseg * 4 <= kWaveShareWaves ? 4 : 2;
}

template <typename T, int NS, int CPL, bool VEC, int CHB, int PK, int XW = kMaxSeg>
static int launch_wave_bwd_c(const snd_bwd_params &p, const WaveGeo &wg, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    const int rg = sh.dim / sh.n_groups;
    const dim3 grid = wave_grid2(sh.batch * sh.n_groups, (rg + CHB * PK - 1) / (CHB * PK)), block(64 * wg.nseg * CHB);
    constexpr bool F32 = std::is_same<T, float>::value;
    constexpr int R = wave_band_rows(NS);
    // (the even-plane variant only where the loads are prefetched: it is their waits that it makes exact)
    const bool even = NS <= 2 && CPL == 1 && PK == 1 && sh.nrows % R == 0 && sh.ncols % (kSeg * CPL) == 0;
    if (even) {
        constexpr bool E = NS <= 2 && CPL == 1 && PK == 1;
        if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, NS, CPL, VEC, true, E, CHB, PK, XW>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_bwd_kernel<T, NS, CPL, VEC, F32, E, CHB, PK, XW>), grid, block, 0, stream, p, wg);
    } else {
        if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, NS, CPL, VEC, true, false, CHB, PK, XW>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_bwd_kernel<T, NS, CPL, VEC, F32, false, CHB, PK, XW>), grid, block, 0, stream, p, wg);
    }
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T, int NS, int CPL, bool VEC>
static int launch_wave_bwd_v(const snd_bwd_params &p, const WaveGeo &wg, hipStream_t stream) {
    const int share = CPL == 1 ? wave_bwd_share(p.f.shape, wg) : 1;
    const int pk = CPL == 1 ? wave_pack(wg, p.f.shape.ncols) : 1;
    // (packed planes always in blocks of four waves: the planes of a wave are added up where the waves of a block are)
    if (pk == 8) return launch_wave_bwd_c<T, NS, CPL, VEC, CPL == 1 ? 4 : 1, CPL == 1 ? 8 : 1>(p, wg, stream);
    if (pk == 4) return launch_wave_bwd_c<T, NS, CPL, VEC, CPL == 1 ? 4 : 1, CPL == 1 ? 4 : 1>(p, wg, stream);
    if (pk == 2) return launch_wave_bwd_c<T, NS, CPL, VEC, CPL == 1 ? 4 : 1, CPL == 1 ? 2 : 1>(p, wg, stream);
    if (share == 4) return launch_wave_bwd_c<T, NS, CPL, VEC, CPL == 1 ? 4 : 1, 1>(p, wg, stream);
    if (share == 2 && wg.nseg > 4) return launch_wave_bwd_c<T, NS, CPL, VEC, (CPL == 1 && NS <= 2) ? 2 : 1, 1, (CPL == 1 && NS <= 2) ? 16 : kMaxSeg>(p, wg, stream);
    if (share == 2) return launch_wave_bwd_c<T, NS, CPL, VEC, CPL == 1 ? 2 : 1, 1>(p, wg, stream);
    return launch_wave_bwd_c<T, NS, CPL, VEC, 1, 1>(p, wg, stream);
}

// One launch per column group of a wide plane, right to left (the stream orders them).
template <typename T, int NS>
static int launch_wave_bwd_wide(const snd_bwd_params &p, WaveGeo wg, float *group_ws, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    constexpr bool F32 = std::is_same<T, float>::value;
    if (!group_ws) return SND_ERR_WORKSPACE;
    wg.bcol = group_ws;
    const dim3 grid = wave_grid2(sh.batch * sh.n_groups, sh.dim / sh.n_groups);
    const int groups = wave_groups(wg.nsegAll);
    for (int q = groups - 1; q >= 0; --q) {
        wg.seg0 = q * kMaxSeg;
        wg.nseg = min(kMaxSeg, wg.nsegAll - wg.seg0);
        wg.extL = q > 0;
        wg.extR = q + 1 < groups;
        const dim3 block(64 * wg.nseg);
        if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, NS, 1, true, true, false, 1, 1, kMaxSeg, true>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_bwd_kernel<T, NS, 1, true, F32, false, 1, 1, kMaxSeg, true>), grid, block, 0, stream, p, wg);
        if (hipGetLastError() != hipSuccess) return SND_ERR_LAUNCH;
    }
    return SND_OK;
}

// A split plane: one launch, two blocks (right half, left half) per pair of channels; the tagged words are zeroed first.
template <typename T, int NS>
static int launch_wave_bwd_split(const snd_bwd_params &p, WaveGeo wg, float *group_ws, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    constexpr bool F32 = std::is_same<T, float>::value;
    constexpr bool K = NS <= 2;                      // (the kernel exists for one and two states)
    const int64_t words = (int64_t)((char *)group_ws - (char *)p.workspace) / 4 + (int64_t)sh.batch * sh.dim * sh.dstate * wave_split_words(wg);
    if (zero_words((int *)p.workspace, words, stream) != SND_OK) return SND_ERR_LAUNCH;
    wg.bcol = group_ws;
    wg.sync = (int *)p.workspace;
    wg.spinLimit = spin_limit();
    wg.nseg = wg.nsegAll / 2;
    wg.seg0 = wg.nseg;                               // (of the right halves; left halves start at segment 0)
    const int rg = sh.dim / sh.n_groups;
    const int units = sh.batch * sh.n_groups * ((rg + 1) / 2);          // channel pairs
    const dim3 grid(2 * 8 * ((units + 7) / 8)), block(64 * (wg.nseg * 2 + 1));   // (two blocks per pair, see the kernel's block mapping; a block's
                                                                              // last wave only fetches what the other half left)
    // (whole bands and whole segments: the instantiation without a branch around a row or a lane, as for whole planes)
    const bool even = sh.nrows % wave_band_rows(NS) == 0 && sh.ncols % kSeg == 0;
    if (even) {
        if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, K ? NS : 1, 1, true, true, true, 2, 1, kMaxSeg, true, true>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_bwd_kernel<T, K ? NS : 1, 1, true, F32, true, 2, 1, kMaxSeg, true, true>), grid, block, 0, stream, p, wg);
    } else {
        if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, K ? NS : 1, 1, true, true, false, 2, 1, kMaxSeg, true, true>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_bwd_kernel<T, K ? NS : 1, 1, true, F32, false, 2, 1, kMaxSeg, true, true>), grid, block, 0, stream, p, wg);
    }
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T>
int launch_wave_bwd_t(const snd_bwd_params &p, float *group_ws, hipStream_t stream) {
    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int N = sh.dstate;
    WaveGeo wg = make_wave_geo(sh.nrows, sh.ncols, N);
    wave_geo_channels(wg, sh.batch, sh.dim, sh.n_groups, sh.delta_dim);
    wg.tag = state_tag(p.f.x_sd, sh);
    if (wg.nsegAll > kMaxSeg)
        return N == 1 ? launch_wave_bwd_wide<T, 1>(p, wg, group_ws, stream) : N == 2 ? launch_wave_bwd_wide<T, 2>(p, wg, group_ws, stream)
             : N == 3 ? launch_wave_bwd_wide<T, 3>(p, wg, group_ws, stream) : launch_wave_bwd_wide<T, 4>(p, wg, group_ws, stream);
    if (group_ws && wave_bwd_split(sh.batch, sh.dim, sh.ncols, N))   // (without a workspace: whole planes, one channel per block)
        return N == 1 ? launch_wave_bwd_split<T, 1>(p, wg, group_ws, stream) : launch_wave_bwd_split<T, 2>(p, wg, group_ws, stream);
    if (wg.cpl == 2) {                               // (N = 1 only)
        const int e = (int)sizeof(T), oe = p.dout_dtype == SND_F32 ? 4 : e;
        const bool vec = wave_aligned_b(f.u, e, 2 * e, {f.u_batch_stride, f.u_d_stride, f.u_h_stride}) &&
                         wave_aligned_b(f.delta, e, 2 * e, {f.delta_batch_stride, f.delta_d_stride, f.delta_h_stride}) &&
                         wave_aligned_b(f.B, e, 2 * e, {f.B_batch_stride, f.B_group_stride, f.B_dstate_stride, f.B_h_stride}) &&
                         wave_aligned_b(f.C, e, 2 * e, {f.C_batch_stride, f.C_group_stride, f.C_dstate_stride, f.C_h_stride}) &&
                         wave_aligned_b(p.dout, oe, 2 * oe, {p.dout_batch_stride, p.dout_d_stride, p.dout_h_stride}) &&
                         wave_aligned_b(p.du, e, 2 * e, {}) && wave_aligned_b(p.ddelta, e, 2 * e, {});
        return vec ? launch_wave_bwd_v<T, 1, 2, true>(p, wg, stream) : launch_wave_bwd_v<T, 1, 2, false>(p, wg, stream);
    }
    return N == 1 ? launch_wave_bwd_v<T, 1, 1, true>(p, wg, stream) : N == 2 ? launch_wave_bwd_v<T, 2, 1, true>(p, wg, stream)
         : N == 3 ? launch_wave_bwd_v<T, 3, 1, true>(p, wg, stream) : launch_wave_bwd_v<T, 4, 1, true>(p, wg, stream);
}

}  // namespace snd
