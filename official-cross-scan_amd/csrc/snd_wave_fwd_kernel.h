// Forward kernel of the 2D-CrossScan selective scan for one to four states per channel (gfx950):
// the row-segment wavefront.
//
// Same mathematics as snd_fwd_kernel.h (reference: selective_scan_fwd_kernel_oflex.cuh:189-346):
//     delta' = softplus(delta + bias)          a = exp2(delta' * A * log2e) * A_decay          bu = B * delta' * u
//     h[i,j] = a*(h[i,j-1] + h[i-1,j] - 0.5*(a[i-1,j] + a[i,j-1])*h[i-1,j-1]) + bu
//     s[i,j] = a*s[i,j-1] + bu                 out = D*u + sum_n C*(h - s + 0.25*bu)
// Mapping: a block owns one (batch, channel); wave w of the block owns columns S*w .. S*w+S-1 of the
// plane (a row segment per row; S = 64, or 128 with two neighbouring columns per lane), the channel's states
// are registers of the lane.
// Along a row the recurrence is first order, h_j = a_j*h_{j-1} + y_j with
//     y_j = a_j*(h[i-1,j] - 0.5*(a[i-1,j] + a[i,j-1])*h[i-1,j-1]) + bu_j
// known from the row above, so a wave resolves its 64 cells of a row with one inclusive scan of the
// affine maps (a_j, y_j) (and (a_j, bu_j) for s) in six DPP steps, then adds the value entering from
// the segment on its left: h = Y + A*h[i, 64w-1].  h[i-1,j] and a[i-1,j] are the lane's own registers
// from the previous row, h[i-1,j-1] and a[i,j-1] come from the lane below (wave_shr:1).
// The segments of a plane form an anti-diagonal wavefront: in step e wave w works on the four rows 4(e-w) ..
// 4(e-w)+3 and reads what wave w-1 left for those rows in LDS in step e-1 (h, s, a of its last column);
// one block barrier per step, no polling.  Global loads are whole rows of 64 consecutive elements per
// wave (one or two full memory lines per instruction), issued a band of rows ahead; nothing is staged
// through LDS.  Saved for the backward: h on the last row of every band of its R rows (x_v) and h, s, a
// entering every segment on every row (x, x_sd), so that the backward can recompute any band of any
// segment on its own.
#pragma once
#include <initializer_list>
#include <type_traits>
#include "snd_device.h"

// Timing studies only (-DSND_WAVE_ABLATE=<bits>, results wrong): 1 no out stores, 2 no block barriers,
// 4 no softplus, 8 no scan, 16 no checkpoint stores, 32 no hand-over through LDS.
#ifndef SND_WAVE_ABLATE
#define SND_WAVE_ABLATE 0
#endif

namespace snd {

// PK > 1: narrow planes packed PK to a wave (wave_pack() in snd_device.h): lane l works on column l % (64 / PK) of
// channel PK * chunk + l / (64 / PK) of the group, every per-channel quantity is a lane's own, and the scan stays
// inside the plane's lanes.  One segment per plane, so nothing is handed over between waves.
// EU: the waves per SIMD the registers are to leave room for (1: no limit asked for).  A plane of 4 to 8 segments
// is a block of as many waves; at the 134 registers the two-state kernel takes by itself (three waves per SIMD) a CU
// holds three such blocks of 4 waves and one of 6 (the second block's waves do not fit the SIMDs the first left half
// full), at 128 registers - a few spilled - four and two.  (The one-state kernel takes 94 and needs no such variant.)
// ONE: the plane is one segment wide (always so with packed planes): nothing is handed over and no LDS is used.  A
// block is kOneWaves independent waves, each with a channel (PK channels) of its own, a quarter of the blocks to hand
// out (measured against blocks of one wave, bf16, one state: 64 x 1536 x 14x14 0.055 -> 0.049 ms, 64 x 768 x 14x14
// 0.035 -> 0.031, 64 x 3072 x 7x7 unchanged at 0.051).
// EXT: the launch works on one column group of a wide plane (wave_wide() in snd_device.h): segments seg0 .. seg0+nseg-1.
// The group's first wave takes what enters it on every row - h, s, a of the column on its left - from global memory,
// where the launch of the group on the left put them (a band's values come with the band's loads, three per state and
// row spread over the lanes of one register) and puts them into the LDS slot a wave on its left would have filled;
// the group's last wave leaves the same for the group on its right.
// The places are those of the column checkpoints the backward reads anyway (x, x_sd of segment seg0 and seg0+nseg).
// EVEN: the plane is a whole number of this kernel's bands high and of 64-column segments wide: no row and no lane is
// skipped, so no branch surrounds a row or its stores and the waits the compiler derives for the prefetched loads are
// exact (as in the backward's instantiation of the same name).  256 planes of 512x512, one state: 0.186 -> 0.174 ms.
template <typename T, int NS, int CPL, bool VEC, bool SAVE, bool OUT32, int PK, int EU, bool ONE, bool EXT = false, bool EVEN = false>
__global__ __launch_bounds__(ONE ? 64 * kOneWaves : 64 * kMaxSeg) __attribute__((amdgpu_waves_per_eu(EU))) void wave_fwd_kernel(const snd_fwd_params p, const WaveGeo wg) {
    static_assert(ONE || PK == 1, "packed planes are one segment wide");
    static_assert(!EVEN || (!ONE && PK == 1 && CPL == 1 && !EXT), "whole planes: several segments, one column per lane");
    static_assert(!EXT || (!ONE && PK == 1 && CPL == 1), "column groups: whole segments, one column per lane");
    constexpr int R = wave_fwd_rows(NS);             // rows per band of this kernel = rows per load group
    constexpr int RC = wave_band_rows(NS);           // spacing of the row checkpoints (the backward's bands)
    static_assert(R % RC == 0, "a band ends on a checkpoint row");
    static_assert(PK == 1 || CPL == 1, "packed planes: one column per lane");
    constexpr int S = 64 / PK;                       // lanes per plane
#ifndef SND_WAVE_RD
#define SND_WAVE_RD 4
#endif
    constexpr int RD = SND_WAVE_RD < R ? SND_WAVE_RD : R;   // rows per wavefront step
    static_assert(R % RD == 0, "a band is a whole number of steps");
    // what a wave leaves for the wave on its right: {h, s, a, -} at its last column, per step parity, row and
    // state.  Wave w writes slot w+1 and reads slot w; slot 0 stays zero (nothing enters the first segment).
    __shared__ float4 sHO[2][kMaxSeg + 1][RD][NS];
    // Only lane 63 of a wave has something to hand over.  Instead of masking the other lanes off (a compare, two
    // exec writes and a branch around every hand-over store), every lane stores: lane 63 to the slot, the others to
    // a word of their own that nobody reads.  One wave instruction costs the wave the same issue time either way.
    __shared__ float4 sDump[ONE ? 1 : 64 * kMaxSeg + RD * NS];

    const snd_shape &sh = p.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = wg.rg, rd = wg.rd;
    int pair, chunk;
    if (!wave_job2(wg, sh.batch * G, pair, chunk)) return;
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), w = ONE ? 0 : wv;
    if (ONE) {                                       // (independent waves: one past the group's last channel just leaves)
        chunk = chunk * kOneWaves + wv;
        if (chunk * PK >= rg) return;
    }
    const int sl = PK > 1 ? lane % S : lane;         // the lane inside its plane
    if (PK > 1) chunk = chunk * PK + lane / S;       // (a lane's own from here on)
    const bool act = PK == 1 || chunk < rg;          // a wave past the last channel of its group repeats it and stores nothing
    if (PK > 1) chunk = min(chunk, rg - 1);
    int b, g;
    wave_pair_split(wg, pair, G, b, g);
    const int c = g * rg + chunk, cd = rd == 1 ? c : c / rd;   // channel of u, of delta
    // channel offsets: in the scalar base pointers, or (packed) in the lanes' offsets
    const int cB = PK > 1 ? 0 : c, chB = PK > 1 ? 0 : chunk, cL = PK > 1 ? c : 0, chL = PK > 1 ? chunk : 0;
    const int nseg = wg.nseg;
    const bool multi = !ONE && nseg > 1;
    if (!ONE && threadIdx.x < 2 * RD * NS) (&sHO[0][0][0][0])[(threadIdx.x / (RD * NS)) * (kMaxSeg + 1) * RD * NS + threadIdx.x % (RD * NS)] = make_float4(0.f, 0.f, 0.f, 0.f);

    // scan origin of this group: memory row = r0m + rs*i; with fh the columns run against the memory order
    const bool fv = p.directions == SND_DIR_CORNERS && (g & 2), fh = p.directions == SND_DIR_CORNERS && (g & 1);
    const int r0m = fv ? H - 1 : 0, rs = fv ? -1 : 1;
    const bool bar = PK == 8 && sl == 0;             // (eight planes per wave) the plane's barrier lane
    const int sg = EXT ? wg.seg0 + w : w;            // this wave's segment of the plane
    const int j0 = PK == 8 ? max(sl - 1, 0) : (sg * kSeg + sl) * CPL;   // this lane's first scan column
    const bool jin = EVEN || (j0 < W && !bar);       // (W is a multiple of CPL: a lane is inside or outside as a whole)
    const int jc = jin ? j0 : W - CPL;
    const int mc = fh ? W - CPL - jc : jc;           // memory column of the lane's lowest address

    float A2[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) A2[n] = p.A[(int64_t)c * p.A_d_stride + (int64_t)n * p.A_dstate_stride];   // (NS == N; scaled below)
    float ld = p.A_decay ? p.A_decay[0] : 1.f;
    const float Dv = p.D ? p.D[c] : 0.f;
    const float bias = p.delta_bias ? p.delta_bias[cd] : 0.f;
    const bool softplus = p.delta_softplus != 0;

    constexpr int ESZ = (int)sizeof(T);
    using OutT = typename std::conditional<OUT32, float, T>::type;
    constexpr int OSZ = (int)sizeof(OutT);
    const T *Bb = (const T *)p.B + (int64_t)b * p.B_batch_stride + (int64_t)g * p.B_group_stride;
    const T *Cb = (const T *)p.C + (int64_t)b * p.C_batch_stride + (int64_t)g * p.C_group_stride;
    const T *ub = (const T *)p.u + (int64_t)b * p.u_batch_stride + (int64_t)(p.u_shared ? chB : cB) * p.u_d_stride;
    const T *db = (const T *)p.delta + (int64_t)b * p.delta_batch_stride + (int64_t)(PK > 1 ? 0 : cd) * p.delta_d_stride;
    if (SAVE && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0 && wg.tag) *(uint32_t *)wg.tag = kTagWave;   // which family wrote this state
    // fused CrossMerge (fp32 out only): the channel adds weight * result to the feature channel it belongs to
    const bool merge = p.merge != 0;
    const float wm = merge && p.merge_weights ? p.merge_weights[c] : 1.f;
    OutT *outb = (OutT *)p.out + (int64_t)b * p.out_batch_stride + (int64_t)(merge ? chB : cB) * p.out_d_stride;
    // byte steps from one scan row to the next (negative when the group scans bottom-up) and column offsets
    const int UhB = (int)p.u_h_stride * ESZ * rs, DhB = (int)p.delta_h_stride * ESZ * rs, BhB = (int)p.B_h_stride * ESZ * rs,
              ChB = (int)p.C_h_stride * ESZ * rs, OhB = (int)p.out_h_stride * OSZ * rs;
    const int64_t BsB = p.B_dstate_stride * ESZ, CsB = p.C_dstate_stride * ESZ;
    const uint32_t colB = (uint32_t)mc * ESZ;
    const uint32_t colU = colB + (uint32_t)(p.u_shared ? chL : cL) * (uint32_t)p.u_d_stride * ESZ,
                   colD = colB + (uint32_t)(PK > 1 ? cd : 0) * (uint32_t)p.delta_d_stride * ESZ,
                   colO = (uint32_t)mc * OSZ + (uint32_t)(merge ? chL : cL) * (uint32_t)p.out_d_stride * OSZ;

    // saved state of this plane set
    const int64_t plane0 = ((int64_t)b * Dm + c) * N;
    float *xv = p.x_v + plane0 * wave_xv_plane(wg) + j0;
    float *xh = SAVE ? p.x + plane0 * wave_x_plane(wg) + (int64_t)sg * 2 * wg.Hp : nullptr;
    float *xs = SAVE ? p.x_sd + plane0 * wave_x_plane(wg) + (int64_t)sg * 2 * wg.Hp : nullptr;
    // (column groups) lane (q*NS + n)*R + r fetches h (q = 0), s (1), a (2) entering segment sg on row r of a band, state n
    constexpr int kExtLanes = 3 * NS * wave_fwd_rows(NS);
    const int el = lane < kExtLanes ? lane : 0, eq = el / (NS * wave_fwd_rows(NS)), er = el % wave_fwd_rows(NS);
    const float *ebase = EXT ? (eq == 1 ? wg.cols : wg.colh) + (plane0 + (el / wave_fwd_rows(NS)) % NS) * wave_x_plane(wg)
                               + (int64_t)sg * 2 * wg.Hp + (eq == 2 ? wg.Hp : 0) : nullptr;
    const bool ext_in = EXT && wg.extL && w == 0, ext_out = EXT && wg.extR && w == wg.nseg - 1;
    float *eoh = EXT ? wg.colh + plane0 * wave_x_plane(wg) + (int64_t)(sg + 1) * 2 * wg.Hp : nullptr;
    float *eos = EXT ? wg.cols + plane0 * wave_x_plane(wg) + (int64_t)(sg + 1) * 2 * wg.Hp : nullptr;

    // Raw bits of a band's rows.  Lanes beyond the last column read the last columns (always in bounds): what they
    // compute only feeds cells further right and is never stored.
    typedef WaveRaw<T, CPL, VEC> Raw;
    struct Stage { Raw u[R], d[R], b[R][NS], c[R][NS]; float e; };
    // Byte offsets advance by one row step per load (one vector add each).  Every band issues the same loads on
    // every path - the wait counters the compiler derives for the prefetch need that - so rows past the end of a
    // ragged last band read the last row again (their step is zero) and are never used.
    auto load_band = [&](Stage &q, int band) {
        const int i0 = band * R;
        const int m0 = mad24(i0, rs, r0m);           // memory row of the band's first scan row
        uint32_t ou = mad24(m0, UhB * rs, colU), od = mad24(m0, DhB * rs, colD), ob = mad24(m0, BhB * rs, colB), oc = mad24(m0, ChB * rs, colB);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            wave_ld(q.u[r], ub, ou);
            wave_ld(q.d[r], db, od);
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                const int sn = n;
                wave_ld(q.b[r][n], (const T *)((const char *)Bb + sn * BsB), ob);
                wave_ld(q.c[r][n], (const T *)((const char *)Cb + sn * CsB), oc);
            }
            const bool more = i0 + r + 1 < H;
            ou += more ? UhB : 0; od += more ? DhB : 0; ob += more ? BhB : 0; oc += more ? ChB : 0;
        }
        if (EXT) q.e = ebase[min(i0 + er, wg.Hp - 1)];   // (by every wave, like the other loads; only the group's first wave uses it)
    };
    // the lane's CPL values in scan order (element e of the raw bits is scan column CPL-1-e when fh)
    auto unpack = [&](const Raw &q, float (&v)[CPL]) {
#pragma unroll
        for (int k = 0; k < CPL; ++k) v[k] = wave_elem(q, k);
        if (CPL == 2 && fh) { const float t = v[0]; v[0] = v[CPL - 1]; v[CPL - 1] = t; }
    };

    float hprev[NS][CPL], aprev[NS][CPL], hdiag[NS];   // h, a of the row above at this lane's columns; h[i-1, S*w-1]
    float ch[NS], cs[NS], ca[NS];                      // (SAVE) what entered this segment on row band*R + lane
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        hdiag[n] = 0.f; ch[n] = 0.f; cs[n] = 0.f; ca[n] = 0.f;
#pragma unroll
        for (int k = 0; k < CPL; ++k) { hprev[n][k] = 0.f; aprev[n][k] = 0.f; }
    }

    const int nFB = (H + R - 1) / R;                 // bands of this kernel
    int step = w;                                    // wavefront step this wave is in (parity selects the LDS buffer)
    const bool hands_over = multi && w + 1 < nseg;
    const bool writer = hands_over && lane == 63;
    float4 *const dump = &sDump[ONE ? 0 : threadIdx.x];

    // one band of rows from `cur`, with the next band's loads issued into `nxt` first
    // (MERGE_: whether out is accumulated with atomics - decided once around the band loop, not at every row's store)
    auto do_band = [&](auto MERGE_, Stage &cur, Stage &nxt, int band) {
        constexpr bool MERGE = decltype(MERGE_)::value;
        __builtin_amdgcn_s_setprio(0);
        load_band(nxt, min(band + 1, nFB - 1));   // unconditionally (the last band once more): a skipped load would leave two
                                                        // paths with different numbers of loads in flight, and the waits follow the smaller
        __builtin_amdgcn_s_setprio(3);              // (the rows at a raised wave priority, the load requests above at the
                                                    // default one: 256 planes of 512x512, one state: 0.192 -> 0.186 ms)
        const int i0 = band * R;
        uint32_t oo = mad24(mad24(i0, rs, r0m), OhB * rs, colO);
        // What the rows need that does not depend on the rows above them - softplus, delta' * u - for the RD rows
        // of a wavefront step at once: independent chains of transcendentals that fill each other's latencies,
        // instead of one such chain in front of every row's scan.  (Per step, not per band: the waves of a block
        // are at different rows of their bands in the same step, and a step lasts as long as its slowest wave.)
        float ub_[R][CPL], dlb[R][CPL], dub_[R][CPL];
        // what the segment on the left left for the rows of a step, fetched together right after the step's barrier
        // (one LDS round trip per step instead of one in front of every row's chain); with four states the
        // registers are needed elsewhere and the rows fetch their own
        constexpr bool HOIST_IN = NS <= 2;
        float4 inb[HOIST_IN ? RD : 1][NS];
        float4 *wr = dump;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // (column groups) what the group on the left left for this step's rows goes where a wave on the left would have
            // put it: the group's first wave fills its own slot, one word per lane, and the rows read it as ever
            if (EXT && r % RD == 0 && ext_in && lane < kExtLanes && er / RD == r / RD)
                ((float *)&sHO[(step + 1) & 1][0][er % RD][(el / wave_fwd_rows(NS)) % NS])[eq] = cur.e;
            if (r % RD == 0 && HOIST_IN && !ONE && !(SND_WAVE_ABLATE & 32)) {
#pragma unroll
                for (int q = 0; q < RD; ++q)
#pragma unroll
                    for (int n = 0; n < NS; ++n) inb[HOIST_IN ? q : 0][n] = sHO[(step + 1) & 1][w][q][n];
            }
            if (r % RD == 0) wr = writer ? &sHO[step & 1][w + 1][0][0] : dump;   // this step's slot (or the lane's own word)
            if (r % RD == 0) {
#pragma unroll
                for (int q = r; q < r + RD; ++q) {
                    unpack(cur.u[q], ub_[q]);
                    unpack(cur.d[q], dlb[q]);
#pragma unroll
                    for (int k = 0; k < CPL; ++k) {
                        const float raw = dlb[q][k] + bias;
                        float dsp;
                        // always evaluated, then selected: a branch around it (the flag is uniform) costs a wave more
                        // issue time than the select, and every model in practice asks for the softplus
                        float sp = (SND_WAVE_ABLATE & 4) ? raw : softplus20(raw, dsp);
                        asm volatile("" : "+v"(sp));
                        dlb[q][k] = softplus ? sp : raw;
                        dub_[q][k] = dlb[q][k] * ub_[q][k];
                    }
                }
            }
            if (EVEN || i0 + r < H) {
                float acc[CPL];
                const float (&u)[CPL] = ub_[r], (&dl)[CPL] = dlb[r], (&du)[CPL] = dub_[r];
#pragma unroll
                for (int k = 0; k < CPL; ++k) acc[k] = 0.f;
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    // what the segment on the left left for this row: h, s, a at column S*w-1
                    const float4 in = ((SND_WAVE_ABLATE & 32) || ONE) ? make_float4(0.f, 0.f, 0.f, 0.f)
                                      : HOIST_IN ? inb[HOIST_IN ? r % RD : 0][n] : sHO[(step + 1) & 1][w][r % RD][n];
                    float a[CPL], bu[CPL], cv[CPL], y[CPL], h[CPL], s[CPL];
                    unpack(cur.b[r][n], bu);
                    unpack(cur.c[r][n], cv);
#pragma unroll
                    for (int k = 0; k < CPL; ++k) {
                        a[k] = fast_exp2(fmaf(dl[k], A2[n], ld));
                        bu[k] = bu[k] * du[k];
                        if (PK == 8) { a[k] = bar ? 0.f : a[k]; bu[k] = bar ? 0.f : bu[k]; }   // the barrier lane's map is (0, 0)
                    }
                    const float a_l = from_prev_lane_pk<PK>(a[CPL - 1], in.z, sl == 0);                // a[i, j-1] of the lane's first column
                    const float h_d = from_prev_lane_pk<PK>(hprev[n][CPL - 1], hdiag[n], sl == 0);     // h[i-1, j-1]
#pragma unroll
                    for (int k = 0; k < CPL; ++k) {
                        const float al = k == 0 ? a_l : a[k > 0 ? k - 1 : 0], hd = k == 0 ? h_d : hprev[n][k > 0 ? k - 1 : 0];
                        const float X = fmaf(-0.5f * (aprev[n][k] + al), hd, hprev[n][k]);
                        y[k] = fmaf(a[k], X, bu[k]);
                    }
                    if (SND_WAVE_ABLATE & 8) {
#pragma unroll
                        for (int k = 0; k < CPL; ++k) { h[k] = y[k]; s[k] = bu[k]; }
                    } else {
                        wave_row_solve<CPL, PK>(a, y, bu, in.x, in.y, h, s);
                    }
#pragma unroll
                    for (int k = 0; k < CPL; ++k) {
                        acc[k] = fmaf(cv[k], fmaf(0.25f, bu[k], h[k] - s[k]), acc[k]);
                        hprev[n][k] = h[k];
                        aprev[n][k] = a[k];
                    }
                    hdiag[n] = in.x;
                    if (!ONE && !(SND_WAVE_ABLATE & 32)) {
                        wr[(r % RD) * NS + n] = make_float4(h[CPL - 1], s[CPL - 1], a[CPL - 1], 0.f);
                    }
                    if (EXT && ext_out && lane == 63) {   // what enters the column group on the right
                        const int64_t o = (int64_t)n * wave_x_plane(wg) + i0 + r;
                        eoh[o] = h[CPL - 1];
                        eoh[o + wg.Hp] = a[CPL - 1];
                        eos[o] = s[CPL - 1];
                    }
                    if (SAVE) {                     // lane r keeps what entered the segment on row r (selects, no branch)
                        const bool mine = lane == r;
                        ch[n] = mine ? in.x : ch[n];
                        cs[n] = mine ? in.y : cs[n];
                        ca[n] = mine ? in.z : ca[n];
                    }
                }
                if (jin && act && (!(SND_WAVE_ABLATE & 1) || acc[0] == 1234.5f)) {
                    float o[CPL];
#pragma unroll
                    for (int k = 0; k < CPL; ++k) o[k] = fmaf(Dv, u[k], acc[k]);
                    if (CPL == 2 && fh) { const float t = o[0]; o[0] = o[CPL - 1]; o[CPL - 1] = t; }
                    if (OUT32 && MERGE) {
#pragma unroll
                        for (int k = 0; k < CPL; ++k) glb_add((float *)((char *)outb + oo) + k, wm * o[k]);
                    } else {
                        wave_st<OutT, CPL, VEC>(outb, oo, o);
                    }
                }
                oo += OhB;
                // row checkpoint: h on the last row of a band of the backward (what its next band starts from; the
                // last row of the plane is nobody's, and a ragged last band leaves none)
                if (r % RC == RC - 1) {
#pragma unroll
                    for (int n = 0; n < NS; ++n) {
                        if (EVEN || (act && !bar && !(SND_WAVE_ABLATE & 16))) {
                            float *dst = xv + (int64_t)n * wave_xv_plane(wg) + (int64_t)(band * (R / RC) + r / RC) * wg.Wp;
                            if (CPL == 2) {
                                const wave_f2 v = {hprev[n][0], hprev[n][CPL - 1]};
                                __builtin_nontemporal_store(v, (wave_f2 *)dst);
                            } else {
                                __builtin_nontemporal_store(hprev[n][0], dst);
                            }
                        }
                    }
                }
            }
            if (multi && r % RD == RD - 1) { if (!(SND_WAVE_ABLATE & 2)) lds_barrier(); ++step; }
        }
        // column checkpoints: lanes 0..R-1 hold what entered the segment on the band's rows
        if (SAVE && w > 0 && lane < R && band * R + lane < wg.Hp && !(SND_WAVE_ABLATE & 16)) {
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                const int64_t o = (int64_t)n * wave_x_plane(wg) + band * R + lane;
                xh[o] = ch[n];
                xh[o + wg.Hp] = ca[n];
                xs[o] = cs[n];
            }
        }
    };

    Stage sA, sB;
    load_band(sA, 0);
    // the per-channel parameters are first used here, behind the first band's loads: a wave of a small plane lives
    // for a few microseconds, and a wait for them in front of those loads would be a round trip of its own
#pragma unroll
    for (int n = 0; n < NS; ++n) A2[n] *= kLog2e;
    ld = __log2f(ld);
    if (!ONE) lds_barrier();                         // the zeroed slot
    if (multi)
        for (int e = 0; e < w; ++e) lds_barrier(); // the waves on the left go first
    if (OUT32 && merge) {
        for (int band = 0; band < nFB; band += 2) {
            do_band(std::true_type{}, sA, sB, band);
            if (band + 1 < nFB) do_band(std::true_type{}, sB, sA, band + 1);
        }
    } else {
        for (int band = 0; band < nFB; band += 2) {
            do_band(std::false_type{}, sA, sB, band);
            if (band + 1 < nFB) do_band(std::false_type{}, sB, sA, band + 1);
        }
    }
    if (multi)
        for (int e = 0; e < nseg - 1 - w; ++e) lds_barrier();
}

// Whether every row of a tensor starts at a multiple of `bytes` (so that a lane's CPL elements come with one access)
static inline bool wave_aligned(const void *ptr, int64_t esz, int bytes, std::initializer_list<int64_t> strides) {
    if ((uintptr_t)ptr % bytes) return false;
    for (int64_t st : strides)
        if ((st * esz) % bytes) return false;
    return true;
}

template <typename T, int NS, int CPL, bool VEC, int PK, int EU, bool ONE>
static int launch_wave_fwd_o(const snd_fwd_params &p, const WaveGeo &wg, hipStream_t stream) {
    const snd_shape &sh = p.shape;
    const int rg = sh.dim / sh.n_groups;
    const int waves = (rg + PK - 1) / PK;            // per (batch, group) pair
    const dim3 grid = wave_grid2(sh.batch * sh.n_groups, ONE ? (waves + kOneWaves - 1) / kOneWaves : waves), block(ONE ? 64 * kOneWaves : 64 * wg.nseg);
    const bool save = p.x != nullptr, out32 = p.out_dtype == SND_F32;
    constexpr bool F = std::is_same<T, float>::value;
    // (whole bands and whole segments, the usual training call - state saved, fp32 out: the instantiation without
    // a branch around a row or a lane)
    constexpr bool kEven = !ONE && PK == 1 && CPL == 1;
    if (kEven && save && out32 && sh.nrows % wave_fwd_rows(NS) == 0 && sh.ncols % kSeg == 0) {
        hipLaunchKernelGGL((wave_fwd_kernel<T, NS, CPL, VEC, true, true, PK, EU, ONE, false, kEven>), grid, block, 0, stream, p, wg);
        return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
    }
    if (save && out32) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, CPL, VEC, true, true, PK, EU, ONE>), grid, block, 0, stream, p, wg);
    else if (save) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, CPL, VEC, true, F, PK, EU, ONE>), grid, block, 0, stream, p, wg);
    else if (out32) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, CPL, VEC, false, true, PK, EU, ONE>), grid, block, 0, stream, p, wg);
    else hipLaunchKernelGGL((wave_fwd_kernel<T, NS, CPL, VEC, false, F, PK, EU, ONE>), grid, block, 0, stream, p, wg);
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T, int NS, int CPL, bool VEC, int PK, int EU>
static int launch_wave_fwd_p(const snd_fwd_params &p, const WaveGeo &wg, hipStream_t stream) {
    constexpr bool kOne = CPL == 1 && EU == 1;       // (the one-segment instantiation exists where it can be asked for)
    if (PK > 1 || (kOne && wg.nseg == 1)) return launch_wave_fwd_o<T, NS, CPL, VEC, PK, EU, (PK > 1 || kOne)>(p, wg, stream);
    return launch_wave_fwd_o<T, NS, CPL, VEC, PK, EU, (PK > 1)>(p, wg, stream);
}

template <typename T, int NS, int CPL, bool VEC>
static int launch_wave_fwd_v(const snd_fwd_params &p, const WaveGeo &wg, hipStream_t stream) {
    const int pk = CPL == 1 ? wave_pack(wg, p.shape.ncols) : 1;
    if (pk == 8) return launch_wave_fwd_p<T, NS, CPL, VEC, CPL == 1 ? 8 : 1, 1>(p, wg, stream);
    if (pk == 4) return launch_wave_fwd_p<T, NS, CPL, VEC, CPL == 1 ? 4 : 1, 1>(p, wg, stream);
    if (pk == 2) return launch_wave_fwd_p<T, NS, CPL, VEC, CPL == 1 ? 2 : 1, 1>(p, wg, stream);
    // Planes of 4 to 8 segments, two states, and more blocks than the GPU holds at three waves per SIMD (three blocks
    // of 4 waves per CU, one of more): the instantiation that leaves room for four waves per SIMD.  Measured
    // 2 x 192 x 200x336, two states: 0.242 -> 0.199 ms; narrower planes lose 10 % to the spills and keep the other.
    constexpr bool kRoomy = NS == 2 && CPL == 1;
    const int64_t blocks = (int64_t)p.shape.batch * p.shape.dim;
    if (kRoomy && wg.nseg >= 4 && blocks > 256 * (wg.nseg == 4 ? 3 : 1)) return launch_wave_fwd_p<T, NS, CPL, VEC, 1, kRoomy ? 4 : 1>(p, wg, stream);
    return launch_wave_fwd_p<T, NS, CPL, VEC, 1, 1>(p, wg, stream);
}

// One launch per column group of a wide plane, left to right (the stream orders them).
template <typename T, int NS>
static int launch_wave_fwd_wide(const snd_fwd_params &p, WaveGeo wg, float *group_ws, hipStream_t stream) {
    const snd_shape &sh = p.shape;
    const bool save = p.x != nullptr, out32 = p.out_dtype == SND_F32;
    constexpr bool F = std::is_same<T, float>::value;
    if (!save && !group_ws) return SND_ERR_WORKSPACE;
    wg.colh = save ? p.x : group_ws;
    wg.cols = save ? p.x_sd : group_ws + (int64_t)sh.batch * sh.dim * sh.dstate * wave_x_plane(wg);
    const dim3 grid = wave_grid2(sh.batch * sh.n_groups, sh.dim / sh.n_groups);
    const int groups = wave_groups(wg.nsegAll);
    for (int q = 0; q < groups; ++q) {
        wg.seg0 = q * kMaxSeg;
        wg.nseg = min(kMaxSeg, wg.nsegAll - wg.seg0);
        wg.extL = q > 0;
        wg.extR = q + 1 < groups;
        const dim3 block(64 * wg.nseg);
        if (save && out32) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, 1, true, true, true, 1, 1, false, true>), grid, block, 0, stream, p, wg);
        else if (save) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, 1, true, true, F, 1, 1, false, true>), grid, block, 0, stream, p, wg);
        else if (out32) hipLaunchKernelGGL((wave_fwd_kernel<T, NS, 1, true, false, true, 1, 1, false, true>), grid, block, 0, stream, p, wg);
        else hipLaunchKernelGGL((wave_fwd_kernel<T, NS, 1, true, false, F, 1, 1, false, true>), grid, block, 0, stream, p, wg);
        if (hipGetLastError() != hipSuccess) return SND_ERR_LAUNCH;
    }
    return SND_OK;
}

template <typename T>
int launch_wave_fwd_t(const snd_fwd_params &p, float *group_ws, hipStream_t stream) {
    const snd_shape &sh = p.shape;
    const int N = sh.dstate;
    WaveGeo wg = make_wave_geo(sh.nrows, sh.ncols, N);
    wave_geo_channels(wg, sh.batch, sh.dim, sh.n_groups, sh.delta_dim);
    wg.tag = state_tag(p.x_sd, sh);
    if (wg.nsegAll > kMaxSeg)
        return N == 1 ? launch_wave_fwd_wide<T, 1>(p, wg, group_ws, stream) : N == 2 ? launch_wave_fwd_wide<T, 2>(p, wg, group_ws, stream)
             : N == 3 ? launch_wave_fwd_wide<T, 3>(p, wg, group_ws, stream) : launch_wave_fwd_wide<T, 4>(p, wg, group_ws, stream);
    if (wg.cpl == 2) {                               // (N = 1 only)
        const int e = (int)sizeof(T), oe = p.out_dtype == SND_F32 ? 4 : e;
        const bool vec = wave_aligned(p.u, e, 2 * e, {p.u_batch_stride, p.u_d_stride, p.u_h_stride}) &&
                         wave_aligned(p.delta, e, 2 * e, {p.delta_batch_stride, p.delta_d_stride, p.delta_h_stride}) &&
                         wave_aligned(p.B, e, 2 * e, {p.B_batch_stride, p.B_group_stride, p.B_dstate_stride, p.B_h_stride}) &&
                         wave_aligned(p.C, e, 2 * e, {p.C_batch_stride, p.C_group_stride, p.C_dstate_stride, p.C_h_stride}) &&
                         wave_aligned(p.out, oe, 2 * oe, {p.out_batch_stride, p.out_d_stride, p.out_h_stride});
        return vec ? launch_wave_fwd_v<T, 1, 2, true>(p, wg, stream) : launch_wave_fwd_v<T, 1, 2, false>(p, wg, stream);
    }
    return N == 1 ? launch_wave_fwd_v<T, 1, 1, true>(p, wg, stream) : N == 2 ? launch_wave_fwd_v<T, 2, 1, true>(p, wg, stream)
         : N == 3 ? launch_wave_fwd_v<T, 3, 1, true>(p, wg, stream) : launch_wave_fwd_v<T, 4, 1, true>(p, wg, stream);
}

}  // namespace snd
