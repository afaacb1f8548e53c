// Forward kernel of the 2D-CrossScan selective scan for gfx950.
//
// Computes what the reference's selective_scan_fwd_kernel computes
// (kernels/selective_nd_scan/include/cusoflex/selective_scan_fwd_kernel_oflex.cuh:189-346):
//     delta' = softplus(delta + bias)                                   (:221-224)
//     a      = exp2(delta' * A * log2e) * A_decay                       (:194-195,245)
//     bu     = B * delta' * u                                           (:225,265)
//     h[i,j] = a*(h[i,j-1] + h[i-1,j] - 0.5*(a[i-1,j]+a[i,j-1])*h[i-1,j-1]) + bu     (:263-272,290)
//     s[i,j] = a*s[i,j-1] + bu                                          (:306-327)
//     out    = D*u + sum_n C*(h - s + 0.25*bu)                          (:226-228,301,334)
// but is organised for CDNA4 rather than translated:
//   * one lane owns one (channel, state) plane and walks it in TE x TE tiles (TE = 8, or 7 for
//     planes that 7 divides better) in plain row-major order, so the recurrence needs no block
//     scans, shuffles or barriers in its dependency chain; a wave holds 64/NP channels x NP
//     states of one (batch, group);
//   * the block stages each B/C tile once in LDS for its 16 channels; the per-pixel work
//     (softplus, delta*u) is done once per pixel while staging, not once per state;
//   * the next tiles' global loads are issued before the current tile is computed (an aligned
//     pair of tiles at a time, so that memory lines are not fetched once per tile);
//   * tiles are always computed in full on zero-padded staging: cells outside the plane only
//     feed cells further right/down, so they never reach a stored value and the inner loops
//     carry no bounds checks;
//   * the sum over states is a DPP reduction inside aligned lane groups;
//   * h at strip bottoms (x_v) doubles as the carry to the next strip and as the backward's row
//     checkpoint; h and s at tile right edges (x, x_sd) are the backward's column checkpoints;
//   * a block either walks a whole plane or (PIPE) one strip of it, the strips of a plane running
//     as a pipeline of blocks one tile apart (few, large planes).
#pragma once
#include <initializer_list>
#include "snd_device.h"

namespace snd {

// VEC: the tile's inputs are staged four columns at a time, one 16-byte (fp32) or 8-byte (16-bit) load per thread and
// tensor instead of one load per element: a quarter of the memory instructions and of their address arithmetic.
// Needs 8x8 tiles, a width that is a multiple of four and tensors whose rows start on such boundaries (fwd_vec_ok).
template <typename T, int NP, bool SAVE, bool PIPE, int TE, bool VEC = false>
__global__ __launch_bounds__(16 * NP) __attribute__((amdgpu_waves_per_eu(NP >= 8 ? 3 : 2, 4))) void fwd_kernel(const snd_fwd_params p, const Geo geo) {
    static_assert(!VEC || TE == 8, "vector staging needs 8x8 tiles");
    constexpr int NCH = VEC ? kTile / 4 / NP : 1;   // (VEC) four-column chunks of a channel's tile per thread
    constexpr int WPB = NP / 4, NT = 16 * NP;      // waves / threads per block
    constexpr int CB = 16;                          // channels per block
    constexpr int NSTR = kTile + 4;                 // per-state pitch: lane n hits banks 4n..4n+3
    constexpr int NBC = 4;                          // B/C elements per thread per tile
    constexpr int NPX = kTile / NP;                 // pixels per thread per tile
    constexpr int DLP = kTile + kCkX;               // delta' tile with one halo row above
    // per-channel pitch of the pixel arrays: 8 mod 32 banks, so that the channels a wave reads at one tile offset
    // sit in different banks (a pitch of 64 put them all in the same one)
    constexpr int PCH = kTile + 8;

    __shared__ __align__(16) float sB[NP * NSTR];
    __shared__ __align__(16) float sC[NP * NSTR];
    __shared__ __align__(16) float sDl[CB * DLP];
    __shared__ __align__(16) float sDu[CB * PCH];    // delta' * u
    __shared__ __align__(16) float sY[CB * PCH];     // sum_n C*(h - s)
    // The bu/4 term of the output, sum_n C*B*delta'*u/4, is delta'*u times a per-pixel sum that all
    // channels share: S/4 = sum_n B*C / 4 is built once per tile (per-wave partial sums at staging, added
    // up by one wave) instead of one multiply-add per state cell.
    __shared__ __align__(16) float sSp[(NP / 4) * kTile], sS[kTile];
    // out of up to four consecutive tiles of a strip (two in the 8-state kernels, whose blocks have
    // less LDS each), flushed together: a 32-byte run per tile row is a partial line write (measured:
    // 13 % of the kernel for the 154 MB of out at B=64, D=192, 56x56), four tiles make whole lines
    constexpr int QT = NP == 16 ? 4 : 2, QC = QT * kCkX;
    constexpr int OROW = NP == 16 ? QC + 8 : QC, OCH = kRows * OROW + (NP == 16 ? 16 : 8);   // padded against bank conflicts
    __shared__ __align__(16) float sOut[CB * OCH];

    const snd_shape &sh = p.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = Dm / G, rd = Dm / sh.delta_dim;
    const int nChunks = (rg + CB - 1) / CB;
    int pair, chunk;
    int I_begin = 0, I_end = geo.nCY;               // strips this block walks
    int *sync = (int *)p.workspace, *progress = nullptr;
    bool dead = false;
    int seen = 0;                                   // last progress count read (strip pipeline)
#ifdef SND_PIPE_TRACE
    int *trace_ = nullptr, trace_wait_ = 0;
#endif
    __shared__ int sDead;                           // (pipelined) a hand-over wait of this block has timed out
    if (SAVE && blockIdx.x == 0 && threadIdx.x == 0 && geo.tag) *(uint32_t *)geo.tag = kTagTile;   // which family wrote this state
    if (PIPE) {
        if (threadIdx.x == 0) sDead = 0;            // ordered before its readers by the barrier in draw_job
        // A job is a band of consecutive strips (one strip each in the fully pipelined case), drawn
        // top band first; band k covers strips ceil(k*nCY/nBands) .. ceil((k+1)*nCY/nBands)-1.
        int band;
        if (!draw_job(sync, sh.batch * G, nChunks, geo.nBands, geo.nQueues, pair, chunk, band)) return;
        const int nPC = sh.batch * G * nChunks;
        const int pc = pair * nChunks + chunk;
        I_begin = (band * geo.nCY + geo.nBands - 1) / geo.nBands;
        I_end = ((band + 1) * geo.nCY + geo.nBands - 1) / geo.nBands;
        (void)nPC;
        progress = sync + kSyncHeader + pc * geo.nCY;
#ifdef SND_PIPE_TRACE
        trace_ = sync + kSyncHeader + 2 * nPC * geo.nCY + 4 * (pc * geo.nCY + I_begin);
        if (threadIdx.x == 0) trace_[0] = (int)wall_clock64();
#endif
    } else if (!xcd_job(blockIdx.x, sh.batch * G, nChunks, pair, chunk)) return;
    const int b = pair / G, g = pair - b * G;
    const int cbase = g * rg + chunk * CB, cend = (g + 1) * rg;
    // scan origin of this group: the scan runs in (i, j) from (0, 0); memory row = mrow(i) = r0m + rs*i,
    // memory column = mcol(j) = c0m + cs*j.  Only the staging loads and the output stores know about it.
    const bool fv = p.directions == SND_DIR_CORNERS && (g & 2), fh = p.directions == SND_DIR_CORNERS && (g & 1);
    const int r0m = fv ? H - 1 : 0, rs = fv ? -1 : 1, c0m = fh ? W - 1 : 0, cs = fh ? -1 : 1;
    auto mrow = [&](int r) { return mad24(r, rs, r0m); };
    auto mcol = [&](int c_) { return mad24(c_, cs, c0m); };

    const int tid = threadIdx.x, wave = tid >> 6;
    const int n = tid % NP, cl = tid / NP;          // state and block-local channel of this lane
    const int c = cbase + cl;
    const bool cvalid = c < cend;
    const bool lvalid = cvalid && n < N;
    const int cc = cvalid ? c : cend - 1, nn = n < N ? n : N - 1;
    const int px = tid & 63, pr = px >> 3, pj = px & 7;   // this thread's pixel in B/C staging

    const float A2 = lvalid ? p.A[(int64_t)cc * p.A_d_stride + (int64_t)nn * p.A_dstate_stride] * kLog2e : 0.f;
    const float ld = p.A_decay ? __log2f(p.A_decay[0]) : 0.f;
    const float Dv = p.D ? p.D[cc] : 0.f;
    const float bias = p.delta_bias ? p.delta_bias[cc / rd] : 0.f;
    const bool softplus = p.delta_softplus != 0;
    // fused CrossMerge: the channel's result is scaled by its weight and added to the merged feature channel
    const bool merge = p.merge != 0;
    const float wm = merge && p.merge_weights ? p.merge_weights[cc] : 1.f;
    const int mshift = merge ? g * rg : 0;          // out channel of channel c is c - mshift

    // per-batch-image base pointers (uniform) and 32-bit offsets inside the image
    const T *Bb = (const T *)p.B + (int64_t)b * p.B_batch_stride + (int64_t)g * p.B_group_stride;
    const T *Cb = (const T *)p.C + (int64_t)b * p.C_batch_stride + (int64_t)g * p.C_group_stride;
    const T *ub = (const T *)p.u + (int64_t)b * p.u_batch_stride;
    const T *db = (const T *)p.delta + (int64_t)b * p.delta_batch_stride;
    const int sh_out = p.out_dtype == SND_F32 ? 2 : 1, esz_out = 1 << sh_out;
    void *outb = (char *)p.out + (int64_t)b * p.out_batch_stride * esz_out;
    // byte offsets inside the batch image: per-lane channel offsets (kept across the tile loop) and
    // row pitches / state strides in bytes
    constexpr int ESZ = (int)sizeof(T);
    const uint32_t cUb = (uint32_t)(p.u_shared ? cc - g * rg : cc) * (uint32_t)p.u_d_stride * ESZ, cDb = (uint32_t)(cc / rd) * (uint32_t)p.delta_d_stride * ESZ;
    const int BhB = (int)p.B_h_stride * ESZ, ChB = (int)p.C_h_stride * ESZ, UhB = (int)p.u_h_stride * ESZ, DhB = (int)p.delta_h_stride * ESZ;
    const int OhB = (int)p.out_h_stride * esz_out;
    // (VEC) the gathered rows of out leave four columns per access if every row of out starts on a four-element boundary
    // (the fused merge adds with atomics, element by element)
    const bool ovec = VEC && !merge && ((uintptr_t)p.out & (uintptr_t)(4 * esz_out - 1)) == 0 && p.out_batch_stride % 4 == 0 &&
                      p.out_d_stride % 4 == 0 && p.out_h_stride % 4 == 0;
    const int64_t BsB = p.B_dstate_stride * ESZ, CsB = p.C_dstate_stride * ESZ;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);   // the wave index as a scalar

    // saved state, tile-major; inside a tile the lanes' values 0-3, then the lanes' values 4-7, so that
    // each 16-byte store or load instruction of a wave covers one contiguous 1 KB run (whole lines):
    //   x_v  [b][strip I][col tile J][half][c][n][4 cols]     x, x_sd  [b][J][I][half][c][n][4 rows]
    const int64_t DN8 = (int64_t)Dm * N * 8;
    const int64_t DN4 = DN8 / 2;                    // the lane's values 0-3 of every lane, then values 4-7
    const int64_t lane_off = ((int64_t)cc * N + nn) * 4;
    float *xv = p.x_v + (int64_t)b * geo.nCY * geo.nCX * DN8 + lane_off;
    float *xh = SAVE ? p.x + (int64_t)b * geo.nCX * geo.nCY * DN8 + lane_off : nullptr;
    float *xs = SAVE ? p.x_sd + (int64_t)b * geo.nCX * geo.nCY * DN8 + lane_off : nullptr;

    const float *myDl = sDl + cl * DLP;
    const float *myDu = sDu + cl * PCH;
    const float *myB = sB + n * NSTR;
    const float *myC = sC + n * NSTR;

    // Raw values of a tile, held in registers between their global load and their LDS commit: as loaded, neither
    // converted nor masked, so that nothing touches them (and waits for them) before the commit.
    // Tiles are loaded in aligned pairs (columns 16m..16m+15, both tiles' loads issued together),
    // so that the two 32-byte halves of each 64-byte run are requested while the memory line is in
    // flight: a line is fetched from HBM twice per strip instead of four times.
    // (Only where it pays and fits: the 16-state whole-plane kernels, which are bandwidth-bound.)
    constexpr bool PAIR = NP == 16;
    constexpr int NHL = (kCkX + NP - 1) / NP;       // halo-row elements per thread (1; 2 with four lanes per channel)
    struct StageE { uint32_t qb[NBC], qc[NBC], qdl[NPX], qu[NPX], qhalo[NHL]; };   // raw: masked and converted at commit
    struct StageV { Raw4<T> vb, vc, vdl[NCH], vu[NCH]; uint32_t qhalo[NHL]; };       // (VEC) one chunk of B and C, NCH of delta and u
    typedef typename std::conditional<VEC, StageV, StageE>::type Stage;
    Stage st0, st1;                                 // tile J uses st0 when J is even (or always), st1 when odd
    float qxv[kCkX], qcorner = 0.f;                 // h of the row above the next tile (from x_v)
    auto load_tile = [&](Stage &q, int I, int J) {
        const int r0 = (SND_TILE_ABLATE & 2) ? 0 : I * TE, j0 = (SND_TILE_ABLATE & 2) ? 0 : J * TE;
        // The thread's element maps are re-derived here from an opaque copy of the thread id, so that
        // they are a few integer ops per tile instead of dozens of registers kept live across the tile.
        SND_THREAD_MAPS(NP);
        // loads are always in bounds (clamped coordinates); commit() zeroes what lies outside the plane
        if constexpr (VEC) {
            // chunk c of a tile = row c / 2, columns 4 * (c % 2) .. + 3; under a mirrored column order the same four
            // memory columns in reverse (the chunk then starts at the memory column of its last scan column)
            auto chunk_off = [&](int c, int hB) {
                const int row = min(r0 + (c >> 1), H - 1), col = min(j0 + (c & 1) * 4, W - 4);
                return (uint32_t)mad24(mrow(row), hB, mcol(col + (fh ? 3 : 0)) * ESZ);
            };
            {
                const int sn = min(t_ >> 4, N - 1), c = t_ & 15;
                ldraw4_b(q.vb, (const T *)((const char *)Bb + sn * BsB), chunk_off(c, BhB));
                ldraw4_b(q.vc, (const T *)((const char *)Cb + sn * CsB), chunk_off(c, ChB));
            }
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                ldraw4_b(q.vdl[k], db, cDb + chunk_off(n + NP * k, DhB));
                ldraw4_b(q.vu[k], ub, cUb + chunk_off(n + NP * k, UhB));
            }
        } else {
            const int row = r0 + pr, col = j0 + pj;
            const int mr = mrow(min(row, H - 1)), mcB = mcol(min(col, W - 1)) * ESZ;
            const uint32_t ob = mad24(mr, BhB, mcB), oc = mad24(mr, ChB, mcB);
#pragma unroll
            for (int k = 0; k < NBC; ++k) {
                const int sn = wave_u + WPB * k, sc = min(sn, N - 1);       // scalar: folded into the base
                q.qb[k] = ldraw_b((const T *)((const char *)Bb + sc * BsB), ob);
                q.qc[k] = ldraw_b((const T *)((const char *)Cb + sc * CsB), oc);
            }
#pragma unroll
            for (int k = 0; k < NPX; ++k) {
                const int pp = n + NP * k;
                const int row_ = r0 + (pp >> 3), col_ = j0 + (pp & 7);
                const int mr_ = mrow(min(row_, H - 1)), mcB_ = mcol(min(col_, W - 1)) * ESZ;
                q.qdl[k] = ldraw_b(db, cDb + mad24(mr_, DhB, mcB_));
                q.qu[k] = ldraw_b(ub, cUb + mad24(mr_, UhB, mcB_));
            }
        }
#pragma unroll
        for (int k = 0; k < NHL; ++k) {     // halo row r0-1 (needed for a[i-1,j] of the strip's first row)
            const int row = r0 - 1, col = j0 + min(n + NP * k, TE - 1);
            q.qhalo[k] = ldraw_b(db, cDb + mad24(mrow(max(row, 0)), DhB, mcol(min(col, W - 1)) * ESZ));
        }
    };
    // the pair of tiles that starts at (I, J), J even (or the single tile when not pairing)
    auto load_pair = [&](int I, int J) {
        load_tile(st0, I, J);
        if (PAIR && J + 1 < geo.nCX) load_tile(st1, I, J + 1);
    };
    // h of the row above tile (I, J), one tile ahead, where this block wrote it itself (whole-plane
    // schedule; every strip of a pipelined band but its first)
    auto prefetch_xv = [&](int I, int J) {
        if ((!PIPE || I > I_begin) && I > 0 && geo.nCX > 1) {   // with one column tile the row comes from registers
            const float *src = xv + ((SND_TILE_ABLATE & 8) ? 1 : ((int64_t)(I - 1) * geo.nCX + J)) * DN8;
            const float4 v0 = ld4_stream(src), v1 = ld4_stream(src + DN4);
            qxv[0] = v0.x; qxv[1] = v0.y; qxv[2] = v0.z; qxv[3] = v0.w;
            qxv[4] = v1.x; qxv[5] = v1.y; qxv[6] = v1.z; qxv[7] = v1.w;
            qcorner = src[J > 0 ? ((TE - 1) >> 2) * DN4 + ((TE - 1) & 3) - DN8 : 0];   // last column of the tile on the left (if any: masked at its use)
        }
    };
    // Strip pipeline: h of the row above tile (I, J), written by the block of strip I-1.  Fetched
    // right before the tile needs it, so that a strip runs one tile behind the strip above.  One wave
    // polls for the hand-over (more pollers only slow the counters down); the rest wait at the barrier.
    // The hand-over goes through a one-row buffer per plane in the workspace, laid out
    // [col tile J][pair k][c][n][2] so that a wave's 8-byte coherent accesses cover whole lines (the
    // x_v checkpoint keeps its own layout and plain streaming stores).  A strip overwrites slot J with
    // its own row once it has consumed it, so the corner h[r0-1][j0-1] is kept from the previous fetch.
    const int64_t DN2 = (int64_t)Dm * N * 2;
    float *hrow = PIPE ? (float *)p.workspace + sync_words((int64_t)sh.batch * G * nChunks, geo.nCY) +
                             (int64_t)b * geo.nCX * DN8 + ((int64_t)cc * N + nn) * 2
                       : nullptr;
    float xv_last = 0.f;
    auto fetch_row_above = [&](int J, float (&row)[kCkX]) {
        const float *src = hrow + (int64_t)J * DN8;
#pragma unroll
        for (int k = 0; k < kCkX; k += 2) ld2_coherent(src + (k >> 1) * DN2, row[k], row[k + 1]);
    };
    float dukeep[NPX];   // D*u of this thread's pixels, for the output phase
    auto commit = [&](const Stage &qr, int I, int J) {
        SND_THREAD_MAPS(NP);
        const int r0 = I * TE, j0 = J * TE;
        float dsp;
        if constexpr (VEC) {
            auto flip4 = [&](float (&v)[4]) {                     // memory order -> scan order under a mirrored column order
                if (fh) { const float a0 = v[0], a1 = v[1]; v[0] = v[3]; v[1] = v[2]; v[2] = a1; v[3] = a0; }
            };
            {
                const int sn = t_ >> 4, c = t_ & 15;
                const bool ok = sn < N && r0 + (c >> 1) < H && j0 + (c & 1) * 4 < W;
                float b4[4], c4[4];
                raw4_to_f32(qr.vb, b4); raw4_to_f32(qr.vc, c4);
                flip4(b4); flip4(c4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { b4[e] = ok ? b4[e] : 0.f; c4[e] = ok ? c4[e] : 0.f; }
                *(float4 *)(sB + sn * NSTR + c * 4) = make_float4(b4[0], b4[1], b4[2], b4[3]);
                *(float4 *)(sC + sn * NSTR + c * 4) = make_float4(c4[0], c4[1], c4[2], c4[3]);
            }
#pragma unroll
            for (int k = 0; k < NCH; ++k) {
                const int c = n + NP * k;
                const bool ok = cvalid && r0 + (c >> 1) < H && j0 + (c & 1) * 4 < W;
                float d4[4], u4[4], du4[4];
                raw4_to_f32(qr.vdl[k], d4); raw4_to_f32(qr.vu[k], u4);
                flip4(d4); flip4(u4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float raw = (ok ? d4[e] : 0.f) + bias;
                    d4[e] = softplus ? softplus20(raw, dsp) : raw;
                    u4[e] = ok ? u4[e] : 0.f;
                    du4[e] = d4[e] * u4[e];
                    dukeep[4 * k + e] = Dv * u4[e];
                }
                *(float4 *)(sDl + cl * DLP + kCkX + c * 4) = make_float4(d4[0], d4[1], d4[2], d4[3]);
                *(float4 *)(sDu + cl * PCH + c * 4) = make_float4(du4[0], du4[1], du4[2], du4[3]);
            }
        } else {
        struct { float qb[NBC], qc[NBC], qdl[NPX], qu[NPX]; } q;
        {   // to fp32; zero outside the plane, the tile (7 x 7 tiles) and the state / channel ranges
            const bool in = pr < TE && pj < TE && r0 + pr < H && j0 + pj < W;
#pragma unroll
            for (int k = 0; k < NBC; ++k) {
                const bool ok = in && wave_u + WPB * k < N;
                q.qb[k] = ok ? raw_to_f32((const T *)nullptr, qr.qb[k]) : 0.f;
                q.qc[k] = ok ? raw_to_f32((const T *)nullptr, qr.qc[k]) : 0.f;
            }
#pragma unroll
            for (int k = 0; k < NPX; ++k) {
                const int pp = n + NP * k;
                const bool ok = cvalid && (pp >> 3) < TE && (pp & 7) < TE && r0 + (pp >> 3) < H && j0 + (pp & 7) < W;
                q.qdl[k] = ok ? raw_to_f32((const T *)nullptr, qr.qdl[k]) : 0.f;
                q.qu[k] = ok ? raw_to_f32((const T *)nullptr, qr.qu[k]) : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < NBC; ++k) {
            const int sn = wave + WPB * k;
            sB[sn * NSTR + px] = q.qb[k];
            sC[sn * NSTR + px] = q.qc[k];
        }
        {
            float part = 0.f;
#pragma unroll
            for (int k = 0; k < NBC; ++k) part = fmaf(q.qb[k], q.qc[k], part);
            sSp[wave * kTile + px] = part;
        }
#pragma unroll
        for (int k = 0; k < NPX; ++k) {
            const int pp = n + NP * k;
            const float raw = q.qdl[k] + bias;
            const float dl = softplus ? softplus20(raw, dsp) : raw;
            sDl[cl * DLP + kCkX + pp] = dl;
            sDu[cl * PCH + pp] = dl * q.qu[k];
            dukeep[k] = Dv * q.qu[k];
        }
        }
#pragma unroll
        for (int k = 0; k < NHL; ++k) {
            const int hj = n + NP * k;
            if (hj < kCkX) {
                const float hv = (hj < TE && cvalid && r0 > 0 && j0 + hj < W) ? raw_to_f32((const T *)nullptr, qr.qhalo[k]) : 0.f;
                const float raw = hv + bias;
                sDl[cl * DLP + hj] = softplus ? softplus20(raw, dsp) : raw;
            }
        }
    };

    load_pair(I_begin, 0);
    prefetch_xv(I_begin, 0);
    for (int I = I_begin; I < I_end; ++I) {
        const int r0 = I * TE;
        float hl[kRows], sl[kRows], al[kRows];      // h, s, a at the column left of the tile
#pragma unroll
        for (int r = 0; r < kRows; ++r) { hl[r] = 0.f; sl[r] = 0.f; al[r] = 0.f; }

        // one tile; `mine` holds its staged inputs, `last_of_pair` says that both register sets are
        // free once it is committed, so the next pair's loads can be issued under its compute
        auto do_tile = [&](const int J, const Stage &mine, const bool last_of_pair) {
            const int j0 = J * TE;
            commit(mine, I, J);
            // first strip of a pipelined band: the row above comes from another block
            const bool handed = PIPE && I == I_begin && I > 0;
            if (handed && wave == 0) {
                strip_wait(progress + I - 1, J + 1, seen, sync, dead, geo.spinLimit SND_TRACE_PASS);
                if (dead && tid == 0) sDead = 1;
            }
            __syncthreads();
            if (wave == 0) {                        // read by the output phase, behind the next barrier
                float t = 0.f;
                if (VEC) {                          // from the committed tile: sum_n B*C of the pixel
#pragma unroll
                    for (int k = 0; k < NP; ++k) t = fmaf(sB[k * NSTR + (tid & 63)], sC[k * NSTR + (tid & 63)], t);
                } else {
#pragma unroll
                    for (int w = 0; w < WPB; ++w) t += sSp[w * kTile + (tid & 63)];
                }
                sS[tid & 63] = 0.25f * t;
            }
            // row above this tile: fetched one tile ahead (taken before the next prefetch reuses the
            // registers), handed over in registers, or - from another block - fetched here
            float hup[kCkX], aup[kCkX];
            float corner = 0.f;                     // h[r0-1][j0-1]
            if (handed) {
                fetch_row_above(J, hup);
                if (lds_peek(&sDead)) {      // the wait timed out: poison everything downstream
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) hup[j] = __builtin_nanf("");
                }
            } else {
                corner = (I > 0 && J > 0) ? qcorner : 0.f;
#pragma unroll
                for (int j = 0; j < kCkX; ++j) hup[j] = (I > 0) ? qxv[j] : 0.f;
            }
            {   // issue the next loads now; they complete while this tile is computed
                int In = I, Jn = J + 1;
                if (Jn == geo.nCX) { Jn = 0; In = I + 1; }
                if (In < I_end) {
                    prefetch_xv(In, Jn);
                    if (last_of_pair) load_pair(In, Jn);
                }
            }
            if (handed) {                           // the corner is the previous fetch's last column
                corner = J > 0 ? xv_last : 0.f;
                xv_last = hup[TE - 1];
            }

            // ---- per-lane tile walk
            // The tile walk runs at the default wave priority and everything around it (stores, epilogue, the next tile's
            // commit and load requests) at a raised one: of a SIMD's three waves the ones with memory instructions to issue
            // go first.  Measured (same box, forward ms): c1 0.497 -> 0.490, c2 0.115 -> 0.109, c3 0.615 -> 0.602,
            // c4 1.177 -> 1.153; the reverse assignment gains half as much.
            __builtin_amdgcn_s_setprio(0);
#pragma unroll
            for (int j = 0; j < kCkX; ++j) aup[j] = (I > 0 && j < TE) ? fast_exp2(fmaf(myDl[j], A2, ld)) : 0.f;

#pragma unroll
            for (int r = 0; r < TE; ++r) {
                float left = hl[r], sleft = sl[r], aleft = al[r];
                float diag = corner;
                corner = hl[r];                     // h[r0+r][j0-1] is the next row's corner
                float y[kCkX];
#pragma unroll
                for (int j4 = 0; j4 < kCkX; j4 += 4) {
                    const float4 vdl = *(const float4 *)(myDl + (r + 1) * kCkX + j4);
                    const float4 vdu = *(const float4 *)(myDu + r * kCkX + j4);
                    const float4 vb = *(const float4 *)(myB + r * kCkX + j4);
                    const float4 vc = *(const float4 *)(myC + r * kCkX + j4);
                    const float adl[4] = {vdl.x, vdl.y, vdl.z, vdl.w};
                    const float adu[4] = {vdu.x, vdu.y, vdu.z, vdu.w};
                    const float ab[4] = {vb.x, vb.y, vb.z, vb.w};
                    const float ac[4] = {vc.x, vc.y, vc.z, vc.w};
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int j = j4 + q;
                        if (j >= TE) { y[j] = 0.f; continue; }   // storage column beyond the tile
                        const float a = fast_exp2(fmaf(adl[q], A2, ld));
                        const float bu = ab[q] * adu[q];
                        const float X = fmaf(-0.5f * (aup[j] + aleft), diag, hup[j]);
                        const float h = fmaf(a, left + X, bu);
                        const float s = fmaf(a, sleft, bu);
                        y[j] = ac[q] * (h - s);
                        diag = hup[j];
                        hup[j] = h; aup[j] = a;
                        left = h; aleft = a; sleft = s;
                    }
                }
                hl[r] = left; sl[r] = sleft; al[r] = aleft;
                if (NP == 16) {
                    // sum over the channel's 16 states; quad q of the lane group ends with columns 2q, 2q+1
                    group_scatter8(y[0], y[1], y[2], y[3], y[4], y[5], y[6], y[7]);
                    if ((n & 3) == 0) *(float2 *)(sY + cl * PCH + r * kCkX + (n >> 1)) = make_float2(y[0], y[1]);
                } else {
                    group_sum4<NP>(y[0], y[1], y[2], y[3]);
                    group_sum4<NP>(y[4], y[5], y[6], y[7]);
                    if (n == 0) {
                        float4 *dst = (float4 *)(sY + cl * PCH + r * kCkX);
                        dst[0] = make_float4(y[0], y[1], y[2], y[3]);
                        dst[1] = make_float4(y[4], y[5], y[6], y[7]);
                    }
                }
            }
            __builtin_amdgcn_s_setprio(3);
            if (geo.nCX == 1 && I + 1 < I_end) {    // the next strip's row above is this tile's last row
#pragma unroll
                for (int j = 0; j < kCkX; ++j) qxv[j] = hup[j];
                qcorner = 0.f;
            }
            // The loads issued at the top of this tile have had the whole tile to arrive.  Waiting for them here, before
            // this tile's stores are issued, keeps every later wait for a loaded value from also covering the
            // acknowledgement of those stores (one counter counts both, and it is not decremented in order across
            // loads and stores).
            __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
            if (lvalid) {
                // row checkpoint / carry to the next strip: h at the strip's last row
                float *dst = xv + ((int64_t)I * geo.nCX + J) * DN8;
                if (!(SND_TILE_ABLATE & 4)) {
                    st4_stream(dst, hup[0], hup[1], hup[2], hup[3]);
                    st4_stream(dst + DN4, hup[4], hup[5], hup[6], hup[7]);
                }
                if (PIPE && I + 1 == I_end && I + 1 < geo.nCY) {   // and the hand-over copy for the block of the strip below
                    float *ho = hrow + (int64_t)J * DN8;
#pragma unroll
                    for (int k = 0; k < kCkX; k += 2) st2_coherent(ho + (k >> 1) * DN2, hup[k], hup[k + 1]);
                }
            }
            const bool hands_over = PIPE && I + 1 == I_end && I + 1 < geo.nCY;
            if (hands_over) strip_stores_done();
            if (lvalid && SAVE && J + 1 < geo.nCX && !(SND_TILE_ABLATE & 4)) {   // column checkpoints: only if a tile follows
                float *dh = xh + ((int64_t)J * geo.nCY + I) * DN8;
                float *ds = xs + ((int64_t)J * geo.nCY + I) * DN8;
                st4_stream(dh, hl[0], hl[1], hl[2], hl[3]);
                st4_stream(dh + DN4, hl[4], hl[5], hl[6], hl[7]);
                st4_stream(ds, sl[0], sl[1], sl[2], sl[3]);
                st4_stream(ds + DN4, sl[4], sl[5], sl[6], sl[7]);
            }
            __syncthreads();
            if (hands_over) strip_signal(progress + I);   // tile J is handed over to the strip below

            // ---- out = D*u + y: finished by the thread that staged the pixel, parked in LDS
            SND_THREAD_MAPS(NP);
            const int jq = J % QT;
            if (geo.nCX <= 2) {                     // narrow planes: nothing to gather, write directly
                const uint32_t cOb = (uint32_t)(cc - mshift) * (uint32_t)p.out_d_stride * esz_out;
#pragma unroll
                for (int k = 0; k < NPX; ++k) {
                    const int pp = VEC ? 4 * (n + NP * (k >> 2)) + (k & 3) : n + NP * k;
                    const int row = r0 + (pp >> 3), col = j0 + (pp & 7);
                    if (cvalid && (pp >> 3) < TE && (pp & 7) < TE && row < H && col < W && !(SND_TILE_ABLATE & 1)) {
                        const float v = fmaf(sDu[cl * PCH + pp], sS[pp], sY[cl * PCH + pp] + dukeep[k]);
                        const uint32_t o = cOb + mad24(mrow(row), OhB, mcol(col) << sh_out);
                        if (merge) glb_add((float *)((char *)outb + o), wm * v);
                        else st_f32_b(outb, o, p.out_dtype, v);
                    }
                }
                return;
            }
            if constexpr (VEC) {
#pragma unroll
                for (int k = 0; k < NCH; ++k) {
                    const int pp = 4 * (n + NP * k);
                    const float4 du4 = *(const float4 *)(sDu + cl * PCH + pp), s4 = *(const float4 *)(sS + pp), y4 = *(const float4 *)(sY + cl * PCH + pp);
                    *(float4 *)(sOut + cl * OCH + (pp >> 3) * OROW + jq * TE + (pp & 7)) =
                        make_float4(wm * fmaf(du4.x, s4.x, y4.x + dukeep[4 * k]), wm * fmaf(du4.y, s4.y, y4.y + dukeep[4 * k + 1]),
                                    wm * fmaf(du4.z, s4.z, y4.z + dukeep[4 * k + 2]), wm * fmaf(du4.w, s4.w, y4.w + dukeep[4 * k + 3]));
                }
            } else {
#pragma unroll
            for (int k = 0; k < NPX; ++k) {
                const int pp = n + NP * k;
                if ((pp >> 3) < TE && (pp & 7) < TE)
                    sOut[cl * OCH + (pp >> 3) * OROW + jq * TE + (pp & 7)] = wm * fmaf(sDu[cl * PCH + pp], sS[pp], sY[cl * PCH + pp] + dukeep[k]);
            }
            }
            // the next commit() does not touch sY; its barrier orders these sY reads against the
            // next tile's sY writes, and the barrier above ordered this tile's LDS reads against it
            if (jq == QT - 1 || J == geo.nCX - 1) {
                // ---- and written out once per QT tiles: consecutive lanes, consecutive columns
                __syncthreads();
                const int c0 = (J - jq) * TE, ncols = min((jq + 1) * TE, W - c0);
                constexpr int PER_CH = kRows * QC;
                if (VEC && ovec) {
                    constexpr int Q4 = QC / 4;      // four-column groups per gathered row
#pragma unroll 1
                    for (int idx = tid; idx < CB * kRows * Q4; idx += 16 * NP) {
                        const int ch = idx / (kRows * Q4), rr = (idx / Q4) & 7, c4 = (idx & (Q4 - 1)) * 4;
                        const int row = r0 + rr;
                        if (row < H && c4 < ncols && cbase + ch < cend && !(SND_TILE_ABLATE & 1)) {
                            const float4 v = *(const float4 *)(sOut + ch * OCH + rr * OROW + c4);
                            float a4[4] = {v.x, v.y, v.z, v.w};
                            if (fh) { a4[0] = v.w; a4[1] = v.z; a4[2] = v.y; a4[3] = v.x; }   // scan order -> memory order
                            const uint32_t o = (uint32_t)(cbase + ch) * (uint32_t)p.out_d_stride * esz_out +
                                               mad24(mrow(row), OhB, mcol(c0 + c4 + (fh ? 3 : 0)) << sh_out);
                            if (p.out_dtype == SND_F32) stg4_b((float *)outb, o, a4);
                            else if (p.out_dtype == SND_BF16) stg4_b((bf16_t *)outb, o, a4);
                            else stg4_b((f16_t *)outb, o, a4);
                        }
                    }
                } else
#pragma unroll 4
                for (int idx = tid; idx < CB * PER_CH; idx += 16 * NP) {
                    const int ch = idx / PER_CH, rr = (idx / QC) & 7, c32 = idx & (QC - 1);
                    const int row = r0 + rr;
                    if (rr < TE && row < H && c32 < ncols && cbase + ch < cend && !(SND_TILE_ABLATE & 1)) {
                        const uint32_t o = (uint32_t)(cbase + ch - mshift) * (uint32_t)p.out_d_stride * esz_out +
                                           mad24(mrow(row), OhB, mcol(c0 + c32) << sh_out);
                        if (merge) glb_add((float *)((char *)outb + o), sOut[ch * OCH + rr * OROW + c32]);
                        else st_f32_b(outb, o, p.out_dtype, sOut[ch * OCH + rr * OROW + c32]);
                    }
                }
                // the next write of sOut is behind the next tile's barriers
            }
        };
        if (PAIR) {
            for (int J = 0; J < geo.nCX; J += 2) {
                const bool single = J + 1 >= geo.nCX;
                do_tile(J, st0, single);
                if (!single) do_tile(J + 1, st1, true);
            }
        } else {
            for (int J = 0; J < geo.nCX; ++J) do_tile(J, st0, true);
        }
    }
#ifdef SND_PIPE_TRACE
    if (PIPE && threadIdx.x == 0) { trace_[1] = (int)wall_clock64(); trace_[2] = trace_wait_; }
#endif
}

template <typename T, int NP, int TE, bool VEC>
static int launch_fwd_te(const snd_fwd_params &p, const Geo &geo, hipStream_t stream) {
    const snd_shape &sh = p.shape;
    const int rg = sh.dim / sh.n_groups;
    const int nChunks = (rg + 15) / 16;
    const int64_t nPC = (int64_t)sh.batch * sh.n_groups * nChunks;
    const int bands = fwd_band_count(p.schedule, (int64_t)sh.batch * sh.n_groups, nChunks, geo.nCY, p.workspace, sh.dstate, geo.nCX);
    if (bands > 0) {
        if (nPC * geo.nCY >= (int64_t)1 << 31) return SND_ERR_SHAPE;
        if (zero_words((int *)p.workspace, sync_words(nPC, geo.nCY), stream) != SND_OK) return SND_ERR_LAUNCH;
        const int grid = (int)(nPC * bands);
        Geo gs = geo;
        gs.spinLimit = spin_limit();
        gs.nBands = bands;
        gs.nQueues = job_queues(sh.batch * sh.n_groups);
        if (p.x != nullptr)
            hipLaunchKernelGGL((fwd_kernel<T, NP, true, true, TE, VEC>), dim3(grid), dim3(16 * NP), 0, stream, p, gs);
        else
            hipLaunchKernelGGL((fwd_kernel<T, NP, false, true, TE, VEC>), dim3(grid), dim3(16 * NP), 0, stream, p, gs);
    } else {
        const int grid = xcd_grid(sh.batch * sh.n_groups, nChunks);
        if (p.x != nullptr)
            hipLaunchKernelGGL((fwd_kernel<T, NP, true, false, TE, VEC>), dim3(grid), dim3(16 * NP), 0, stream, p, geo);
        else
            hipLaunchKernelGGL((fwd_kernel<T, NP, false, false, TE, VEC>), dim3(grid), dim3(16 * NP), 0, stream, p, geo);
    }
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

// Whether a call can stage four columns per load (fwd_kernel's VEC): every row of u, delta, B and C must start on a
// four-element boundary (16 bytes of fp32, 8 bytes of 16-bit values); a state's plane of B / C must lie within 2^31
// bytes of the first (the state offset is per lane there).
inline bool fwd_vec_ok(const snd_fwd_params &f) {
    const snd_shape &sh = f.shape;
    const int e = sh.in_dtype == SND_F32 ? 4 : 2;
    if (sh.ncols % 4 != 0) return false;
    auto ok = [&](const void *ptr, std::initializer_list<int64_t> strides) {
        if (((uintptr_t)ptr & (uintptr_t)(4 * e - 1)) != 0) return false;
        for (int64_t s : strides)
            if (s % 4 != 0) return false;
        return true;
    };
    const int64_t span = (int64_t)(sh.dstate - 1) * e;
    if (span * f.B_dstate_stride + (int64_t)sh.nrows * f.B_h_stride * e >= ((int64_t)1 << 31) ||
        span * f.C_dstate_stride + (int64_t)sh.nrows * f.C_h_stride * e >= ((int64_t)1 << 31))
        return false;
    return ok(f.u, {f.u_batch_stride, f.u_d_stride, f.u_h_stride}) && ok(f.delta, {f.delta_batch_stride, f.delta_d_stride, f.delta_h_stride}) &&
           ok(f.B, {f.B_batch_stride, f.B_group_stride, f.B_dstate_stride, f.B_h_stride}) &&
           ok(f.C, {f.C_batch_stride, f.C_group_stride, f.C_dstate_stride, f.C_h_stride});
}

template <typename T, int NP>
static int launch_fwd_np(const snd_fwd_params &p, hipStream_t stream) {
    Geo geo = make_geo(p.shape.nrows, p.shape.ncols);
    geo.tag = state_tag(p.x_sd, p.shape);
    if (geo.te == 7) return launch_fwd_te<T, NP, 7, false>(p, geo, stream);
    return fwd_vec_ok(p) ? launch_fwd_te<T, NP, 8, true>(p, geo, stream) : launch_fwd_te<T, NP, 8, false>(p, geo, stream);
}

// One instantiation per input dtype, each in its own translation unit.
template <typename T>
int launch_fwd_t(const snd_fwd_params &p, hipStream_t stream) {
    // (four lanes per channel for N <= 4 work here too, but measure slower than eight: one-wave blocks
    // with 16 staged pixels per thread; the backward does use them)
    return p.shape.dstate > 8 ? launch_fwd_np<T, 16>(p, stream) : launch_fwd_np<T, 8>(p, stream);
}

}  // namespace snd
