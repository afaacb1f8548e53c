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
// Organisation (not a translation): the same lane = one (channel, state) plane, 8x8 tile walk as the
// forward, in reverse.  For each tile a lane recomputes h from the forward's checkpoints (row above
// from x_v, column to the left from x, s from x_sd) into 64 registers, then sweeps the tile
// bottom-right to top-left.  The adjoint row handed to the strip above goes through a private
// global scratch row; the column handed to the tile on the left stays in registers.  dB/dC are
// reduced over the block's 16 channels with LDS atomics and leave the block once per tile;
// du/ddelta are reduced over states by DPP and finished once per pixel by the thread that staged it.
// As in the forward, tiles are computed in full on zero-padded staging (dout = B = C = 0 outside
// the plane makes every adjoint there exactly zero), so the inner loops have no bounds checks.
#include "snd_device.h"

namespace snd {

__device__ __forceinline__ void lds_add(float *p, float v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void glb_add(float *p, float v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// v_permlane32_swap: upper 32 lanes of a <-> lower 32 lanes of b.  v_permlane16_swap: odd 16-lane
// rows of a <-> even rows of b.  After either swap, a + b is the pair-sum of the value the lane keeps.
__device__ __forceinline__ void swap32(float &a, float &b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap16(float &a, float &b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// Sum v[0..7] over the four 16-lane rows of a wave (= its four channels when a row holds the 16
// states of one channel).  Row q of the wave ends up with the totals of v[2q] and v[2q+1]:
// a reduce-scatter, 12 swaps + 12 adds for 8 values instead of 16 for a broadcast sum.
__device__ __forceinline__ void rows_reduce8(const float (&v)[8], float &w0, float &w1) {
    float t[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) { float a = v[k], b = v[k + 4]; swap32(a, b); t[k] = a + b; }
    { float a = t[0], b = t[2]; swap16(a, b); w0 = a + b; }
    { float a = t[1], b = t[3]; swap16(a, b); w1 = a + b; }
}

template <int NP>
__global__ __launch_bounds__(16 * NP) void bwd_kernel(const snd_bwd_params p, const Geo geo) {
    constexpr int WPB = NP / 4;                     // waves per block
    constexpr int CB = 16;                          // channels per block
    constexpr int NSTR = kTile + 4;
    constexpr int NBC = 4;
    constexpr int NPX = kTile / NP;
    constexpr int HG = 10, DLP = HG * HG;           // delta' on the tile plus a one-cell halo
    constexpr int NHALO = 36, NHK = (NHALO + NP - 1) / NP;

    // NP == 16: a wave's four channels are reduced in registers (rows_reduce8) and every wave owns
    // a partial dB/dC tile, written with plain stores.  NP == 8: one shared tile, LDS atomics.
    constexpr int NPART = (NP == 16) ? WPB : 1;
    extern __shared__ __align__(16) float smem[];
    float *sB = smem;                               // [NP][NSTR]
    float *sC = sB + NP * NSTR;
    float *sdB = sC + NP * NSTR;                    // [NPART][NP][NSTR]
    float *sdC = sdB + NPART * NP * NSTR;
    float *sDl = sdC + NPART * NP * NSTR;           // [CB][DLP]
    float *sDu = sDl + CB * DLP;                    // [CB][kTile] delta' * u
    float *sU = sDu + CB * kTile;
    float *sDo = sU + CB * kTile;                   // dout
    float *sSg = sDo + CB * kTile;                  // d softplus / d raw
    float *sQ = sSg + CB * kTile;                   // sum_n dbu*B
    float *sP = sQ + CB * kTile;                    // sum_n A*da*a
    float *sRed = sP + CB * kTile;                  // [WPB]

    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups, dt = sh.in_dtype;
    const int rg = Dm / G, rd = Dm / sh.delta_dim;
    const int nChunks = (rg + CB - 1) / CB;
    int pair, chunk;
    if (!xcd_job(blockIdx.x, sh.batch * G, nChunks, pair, chunk)) return;
    const int b = pair / G, g = pair - b * G;
    const int cbase = g * rg + chunk * CB, cend = (g + 1) * rg;

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

    const int64_t offB = (int64_t)b * f.B_batch_stride + (int64_t)g * f.B_group_stride;
    const int64_t offC = (int64_t)b * f.C_batch_stride + (int64_t)g * f.C_group_stride;
    const int64_t offU = (int64_t)b * f.u_batch_stride + (int64_t)cc * f.u_d_stride;
    const int64_t offD = (int64_t)b * f.delta_batch_stride + (int64_t)(cc / rd) * f.delta_d_stride;
    const int64_t offDo = (int64_t)b * p.dout_batch_stride + (int64_t)cc * p.dout_d_stride;
    const int64_t offG = ((int64_t)b * Dm + cc) * H * W;             // du, ddelta: dense [b, c, H, W]
    float *dBg = p.dB + ((int64_t)b * G + g) * N * H * W;            // dense [b, g, N, H, W]
    float *dCg = p.dC + ((int64_t)b * G + g) * N * H * W;

    // saved state and scratch, (channel, state) innermost (same layouts as the forward writes):
    //   x_v [b][strip][col][c][n]   x, x_sd [b][col tile][row][c][n]   scratch G row [b][col][c][n]
    const int64_t DN = (int64_t)Dm * N;
    const int64_t lane_off = (int64_t)cc * N + nn;
    const float *xv = f.x_v + (int64_t)b * geo.nCY * geo.Wp * DN + lane_off;
    const float *xh = f.x + (int64_t)b * geo.nCX * geo.Hp * DN + lane_off;
    const float *xs = f.x_sd + (int64_t)b * geo.nCX * geo.Hp * DN + lane_off;
    float *gdown = (float *)p.workspace + (int64_t)b * geo.Wp * DN + lane_off;

    const float *myDl = sDl + cl * DLP;
    const float *myDu = sDu + cl * kTile;
    const float *myDo = sDo + cl * kTile;
    const float *myB = sB + n * NSTR;
    const float *myC = sC + n * NSTR;
    float *mydB = sdB + (NP == 16 ? wave * NP * NSTR : 0) + n * NSTR;
    float *mydC = sdC + (NP == 16 ? wave * NP * NSTR : 0) + n * NSTR;
    const int qrow = (tid & 63) >> 4;               // 16-lane row of this lane inside its wave

    if (NP != 16)
        for (int i = tid; i < NP * NSTR; i += 16 * NP) { sdB[i] = 0.f; sdC[i] = 0.f; }

    // ---- register staging of one tile's raw inputs (global loads issued one tile ahead)
    float qb[NBC], qc[NBC], qdl[NPX], qu[NPX], qdo[NPX], qh[NHK];
    auto prefetch = [&](int I, int J) {
        const int r0 = I * kRows, j0 = J * kCkX;
        {
            const int row = r0 + pr, col = j0 + pj;
            const bool in = row < H && col < W;
#pragma unroll
            for (int k = 0; k < NBC; ++k) {
                const int sn = wave + WPB * k;
                const bool ok = in && sn < N;
                qb[k] = ok ? ld_f32(f.B, offB + (int64_t)sn * f.B_dstate_stride + (int64_t)row * f.B_h_stride + col, dt) : 0.f;
                qc[k] = ok ? ld_f32(f.C, offC + (int64_t)sn * f.C_dstate_stride + (int64_t)row * f.C_h_stride + col, dt) : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < NPX; ++k) {
            const int pp = n + NP * k;
            const int row = r0 + (pp >> 3), col = j0 + (pp & 7);
            const bool ok = cvalid && row < H && col < W;
            qdl[k] = ok ? ld_f32(f.delta, offD + (int64_t)row * f.delta_h_stride + col, dt) : 0.f;
            qu[k] = ok ? ld_f32(f.u, offU + (int64_t)row * f.u_h_stride + col, dt) : 0.f;
            qdo[k] = ok ? ld_f32(p.dout, offDo + (int64_t)row * p.dout_h_stride + col, p.dout_dtype) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < NHK; ++k) {   // the 36 halo cells of the 10x10 delta' grid
            const int hidx = n + NP * k;
            int rr, jj;
            if (hidx < 10) { rr = 0; jj = hidx; }
            else if (hidx < 20) { rr = 9; jj = hidx - 10; }
            else if (hidx < 28) { rr = hidx - 19; jj = 0; }
            else { rr = hidx - 27; jj = 9; }
            const int row = r0 - 1 + rr, col = j0 - 1 + jj;
            const bool ok = hidx < NHALO && cvalid && row >= 0 && row < H && col >= 0 && col < W;
            qh[k] = ok ? ld_f32(f.delta, offD + (int64_t)row * f.delta_h_stride + col, dt) : 0.f;
        }
    };
    auto commit = [&]() {
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
            sDl[cl * DLP + ((pp >> 3) + 1) * HG + (pp & 7) + 1] = dl;
            sDu[cl * kTile + pp] = dl * qu[k];
            sU[cl * kTile + pp] = qu[k];
            sDo[cl * kTile + pp] = qdo[k];
            sSg[cl * kTile + pp] = dsp;
        }
#pragma unroll
        for (int k = 0; k < NHK; ++k) {
            const int hidx = n + NP * k;
            int rr, jj;
            if (hidx < 10) { rr = 0; jj = hidx; }
            else if (hidx < 20) { rr = 9; jj = hidx - 10; }
            else if (hidx < 28) { rr = hidx - 19; jj = 0; }
            else { rr = hidx - 27; jj = 9; }
            const float raw = qh[k] + bias;
            float dsp;
            if (hidx < NHALO) sDl[cl * DLP + rr * HG + jj] = softplus ? softplus20(raw, dsp) : raw;
        }
    };
#define DL(r, j) myDl[((r) + 1) * HG + (j) + 1]
#define AEXP(r, j) fast_exp2(fmaf(DL(r, j), A2, ld))

    float dA_acc = 0.f, dec_acc = 0.f;              // per lane: sum delta'*da*a, sum da*a
    float dD_acc = 0.f, dbias_acc = 0.f;            // per thread, for its channel's staged pixels

    prefetch(geo.nCY - 1, geo.nCX - 1);
    for (int I = geo.nCY - 1; I >= 0; --I) {
        const int r0 = I * kRows;
        float GR[kRows], GsR[kRows];                // G, Gs at the column right of the tile
        float GRc = 0.f;                            // G[r0+8][j0+8]
#pragma unroll
        for (int r = 0; r < kRows; ++r) { GR[r] = 0.f; GsR[r] = 0.f; }

        for (int J = geo.nCX - 1; J >= 0; --J) {
            const int j0 = J * kCkX;
            commit();
            __syncthreads();
            {
                int In = I, Jn = J - 1;
                if (Jn < 0) { Jn = geo.nCX - 1; In = I - 1; }
                if (In >= 0) prefetch(In, Jn);
            }

            // ---- checkpoints and carried adjoints of this tile
            float hu[kCkX], hlft[kRows], slft[kRows], hc = 0.f;
            float Gd[kCkX];
            if (I > 0) {
                const float *src = xv + ((int64_t)(I - 1) * geo.Wp + j0) * DN;
#pragma unroll
                for (int j = 0; j < kCkX; ++j) hu[j] = src[j * DN];
                if (J > 0) hc = src[-DN];
            } else {
#pragma unroll
                for (int j = 0; j < kCkX; ++j) hu[j] = 0.f;
            }
            if (J > 0) {
                const float *sh_ = xh + ((int64_t)(J - 1) * geo.Hp + r0) * DN;
                const float *ss_ = xs + ((int64_t)(J - 1) * geo.Hp + r0) * DN;
#pragma unroll
                for (int r = 0; r < kRows; ++r) { hlft[r] = sh_[r * DN]; slft[r] = ss_[r * DN]; }
            } else {
#pragma unroll
                for (int r = 0; r < kRows; ++r) { hlft[r] = 0.f; slft[r] = 0.f; }
            }
            if (I + 1 < geo.nCY && lvalid) {
                const float *src = gdown + (int64_t)j0 * DN;
#pragma unroll
                for (int j = 0; j < kCkX; ++j) Gd[j] = src[j * DN];
            } else {
#pragma unroll
                for (int j = 0; j < kCkX; ++j) Gd[j] = 0.f;
            }
            const float gd_old0 = Gd[0];            // G[r0+8][j0]: the corner of the tile on the left
            float Gd8 = GRc;

            // ---- recompute h on the tile
            float hT[kRows][kCkX];
            {
                float aprev[kCkX];
#pragma unroll
                for (int j = 0; j < kCkX; ++j) aprev[j] = AEXP(-1, j);
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    float al = AEXP(r, -1);
                    float left = hlft[r];
                    float diag = (r == 0) ? hc : hlft[r - 1 < 0 ? 0 : r - 1];
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) {
                        const float a = AEXP(r, j);
                        const float bu = myB[r * kCkX + j] * myDu[r * kCkX + j];
                        const float up = (r == 0) ? hu[j] : hT[r - 1 < 0 ? 0 : r - 1][j];
                        const float X = fmaf(-0.5f * (aprev[j] + al), diag, up);
                        const float h = fmaf(a, left + X, bu);
                        hT[r][j] = h;
                        diag = up; left = h; al = a; aprev[j] = a;
                    }
                }
            }

            // ---- reverse sweep
            float adn[kCkX];
#pragma unroll
            for (int j = 0; j < kCkX; ++j) adn[j] = AEXP(kRows, j);
#pragma unroll
            for (int r = kRows - 1; r >= 0; --r) {
                float arow[kCkX + 1], bu[kCkX], s[kCkX];
#pragma unroll
                for (int j = 0; j <= kCkX; ++j) arow[j] = AEXP(r, j);
                {
                    float sp = slft[r];
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) {
                        bu[j] = myB[r * kCkX + j] * myDu[r * kCkX + j];
                        sp = fmaf(arow[j], sp, bu[j]);
                        s[j] = sp;
                    }
                }
                float Gr = GR[r], Gsr = GsR[r], Gdiag = Gd8;
                float q[kCkX], pp_[kCkX], vB[kCkX], vC[kCkX];
#pragma unroll
                for (int j = kCkX - 1; j >= 0; --j) {
                    const float dov = myDo[r * kCkX + j];
                    const float Bv = myB[r * kCkX + j], Cv = myC[r * kCkX + j];
                    const float dyC = dov * Cv;
                    const float a = arow[j];
                    const float g_ = fmaf(-0.5f * (arow[j + 1] + adn[j]), Gdiag, dyC + Gr + Gd[j]);
                    const float gs = Gsr - dyC;
                    const float dbu = fmaf(0.25f, dyC, g_ + gs);
                    q[j] = dbu * Bv;
                    vB[j] = dbu * myDu[r * kCkX + j];
                    const float hb = hT[r][j] - bu[j], sb = s[j] - bu[j];
                    vC[j] = dov * fmaf(0.25f, bu[j], hb - sb);
                    const float h_l = (j == 0) ? hlft[r] : hT[r][j - 1 < 0 ? 0 : j - 1];
                    const float h_u = (r == 0) ? hu[j] : hT[r - 1 < 0 ? 0 : r - 1][j];
                    const float cross = fmaf(Gd[j], h_l, Gr * h_u);
                    const float da = fmaf(-0.5f * a, cross, fmaf(g_, hb, gs * sb));
                    pp_[j] = Av * da;
                    dA_acc = fmaf(DL(r, j), da, dA_acc);
                    dec_acc += da;
                    const float Gn = a * g_;
                    Gdiag = Gd[j];
                    Gd[j] = Gn;
                    Gr = Gn;
                    Gsr = a * gs;
                }
                Gd8 = GR[r];                        // G[r][j0+8]: diagonal neighbour for the row above
                GR[r] = Gr;                         // G[r][j0]: right neighbour for the tile on the left
                GsR[r] = Gsr;
#pragma unroll
                for (int j = 0; j < kCkX; ++j) adn[j] = arow[j];
                if (NP == 16) {                     // sum over the wave's 4 channels, then one plain store
                    float b0, b1, c0, c1;
                    rows_reduce8(vB, b0, b1);
                    rows_reduce8(vC, c0, c1);
                    *(float2 *)(mydB + r * kCkX + 2 * qrow) = make_float2(b0, b1);
                    *(float2 *)(mydC + r * kCkX + 2 * qrow) = make_float2(c0, c1);
                } else {
#pragma unroll
                    for (int j = 0; j < kCkX; ++j) { lds_add(mydB + r * kCkX + j, vB[j]); lds_add(mydC + r * kCkX + j, vC[j]); }
                }
#pragma unroll
                for (int j = 0; j < kCkX; ++j) { q[j] = group_sum<NP>(q[j]); pp_[j] = group_sum<NP>(pp_[j]); }
                if (n == 0) {
                    float4 *dq = (float4 *)(sQ + cl * kTile + r * kCkX);
                    float4 *dp = (float4 *)(sP + cl * kTile + r * kCkX);
                    dq[0] = make_float4(q[0], q[1], q[2], q[3]);
                    dq[1] = make_float4(q[4], q[5], q[6], q[7]);
                    dp[0] = make_float4(pp_[0], pp_[1], pp_[2], pp_[3]);
                    dp[1] = make_float4(pp_[4], pp_[5], pp_[6], pp_[7]);
                }
            }
            GRc = gd_old0;
            if (I > 0 && lvalid) {                  // adjoint row for the strip above
                float *dst = gdown + (int64_t)j0 * DN;
#pragma unroll
                for (int j = 0; j < kCkX; ++j) dst[j * DN] = Gd[j];
            }
            __syncthreads();

            // ---- once per pixel: du, ddelta (thread that staged the pixel), dD, ddelta_bias
#pragma unroll
            for (int k = 0; k < NPX; ++k) {
                const int pp = n + NP * k;
                const int row = r0 + (pp >> 3), col = j0 + (pp & 7);
                const float qv = sQ[cl * kTile + pp], pv = sP[cl * kTile + pp];
                const float dl = sDl[cl * DLP + ((pp >> 3) + 1) * HG + (pp & 7) + 1];
                const float uv = sU[cl * kTile + pp], dov = sDo[cl * kTile + pp], sg = sSg[cl * kTile + pp];
                const float duv = fmaf(Dv, dov, dl * qv);
                const float ddl = fmaf(uv, qv, pv) * sg;
                dD_acc = fmaf(dov, uv, dD_acc);
                dbias_acc += ddl;
                if (cvalid && row < H && col < W) {
                    st_f32(p.du, offG + (int64_t)row * W + col, dt, duv);
                    st_f32(p.ddelta, offG + (int64_t)row * W + col, dt, ddl);
                }
            }
            // ---- dB, dC of this tile leave the block (summed over its channels)
            {
                const int row = r0 + pr, col = j0 + pj;
                const bool in = row < H && col < W;
#pragma unroll
                for (int k = 0; k < NBC; ++k) {
                    const int sn = wave + WPB * k;
                    float tb = 0.f, tc = 0.f;
#pragma unroll
                    for (int w = 0; w < NPART; ++w) {
                        tb += sdB[w * NP * NSTR + sn * NSTR + px];
                        tc += sdC[w * NP * NSTR + sn * NSTR + px];
                    }
                    if (in && sn < N) {
                        const int64_t o = (int64_t)sn * H * W + (int64_t)row * W + col;
                        glb_add(dBg + o, tb);
                        glb_add(dCg + o, tc);
                    }
                    if (NP != 16) { sdB[sn * NSTR + px] = 0.f; sdC[sn * NSTR + px] = 0.f; }
                }
            }
        }
    }
#undef DL
#undef AEXP

    // ---- per-lane / per-channel sums leave the kernel
    if (lvalid) glb_add(p.dA + (int64_t)c * N + n, dA_acc);
    dD_acc = group_sum<NP>(dD_acc);
    dbias_acc = group_sum<NP>(dbias_acc);
    if (n == 0 && cvalid) {
        if (p.dD) glb_add(p.dD + c, dD_acc);
        if (p.ddelta_bias) glb_add(p.ddelta_bias + c, dbias_acc);
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

template <int NP>
static int launch_bwd_np(const snd_bwd_params &p, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    const Geo geo = make_geo(sh.nrows, sh.ncols);
    const int rg = sh.dim / sh.n_groups;
    const int nChunks = (rg + 15) / 16;
    const int grid = xcd_grid(sh.batch * sh.n_groups, nChunks);
    constexpr int WPB = NP / 4, NSTR = kTile + 4, NPART = (NP == 16) ? WPB : 1;
    constexpr size_t lds = sizeof(float) * ((2 + 2 * NPART) * NP * NSTR + 16 * 100 + 6 * 16 * kTile + WPB);
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void *)bwd_kernel<NP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return SND_ERR_LAUNCH;
        configured = true;
    }
    hipLaunchKernelGGL((bwd_kernel<NP>), dim3(grid), dim3(16 * NP), lds, stream, p, geo);
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

int launch_bwd(const snd_bwd_params &p, hipStream_t stream) {
    return p.f.shape.dstate > 8 ? launch_bwd_np<16>(p, stream) : launch_bwd_np<8>(p, stream);
}

}  // namespace snd
