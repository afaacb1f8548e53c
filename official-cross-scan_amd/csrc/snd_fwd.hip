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
//   * one lane owns one (channel, state) plane and walks it tile by tile in plain row-major
//     order, so the recurrence needs no block scans, shuffles or barriers in its dependency
//     chain; a wave holds 64/NP channels x NP states of one (batch, group);
//   * the block (4 waves) stages each B/C tile once in LDS for all of its channels, and the
//     per-pixel work (softplus, delta*u) is done once per pixel while staging, not per state;
//   * the sum over states is a DPP reduction inside aligned lane groups;
//   * h at strip bottoms (x_v) doubles as the carry to the next strip and as the backward's row
//     checkpoint; h and s at tile right edges (x, x_sd) are the backward's column checkpoints.
#include "snd_device.h"

namespace snd {

template <typename T, typename TO, int NP, int WPB, int TC, bool SAVE>
__global__ __launch_bounds__(WPB * kWave) void fwd_kernel(const snd_fwd_params p, const Geo geo) {
    constexpr int R = kRows;
    constexpr int CPW = kWave / NP;                 // channels per wave
    constexpr int CB = CPW * WPB;                   // channels per block
    constexpr int kThreads = WPB * kWave;
    constexpr int NSTR = R * TC + 4;                // per-state pitch: lane n hits banks 4n..4n+3
    constexpr int NG = TC / kCkX;                   // column-checkpoint groups per tile
    static_assert(TC % kCkX == 0, "tile width must be a multiple of the checkpoint spacing");

    __shared__ __align__(16) float sB[NP * NSTR];
    __shared__ __align__(16) float sC[NP * NSTR];
    __shared__ __align__(16) float sDl[CB * (R + 1) * TC];   // delta' with one halo row above
    __shared__ __align__(16) float sDu[CB * R * TC];         // delta' * u
    __shared__ __align__(16) float sY[CB * R * TC];          // sum_n C*(h - s + bu/4)

    const snd_shape &sh = p.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = Dm / G, rd = Dm / sh.delta_dim;
    const int nChunks = (rg + CB - 1) / CB;
    int pair, chunk;
    if (!xcd_job(blockIdx.x, sh.batch * G, nChunks, pair, chunk)) return;
    const int b = pair / G, g = pair - b * G;
    const int cbase = g * rg + chunk * CB, cend = (g + 1) * rg;

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int n = lane % NP, cl = wave * CPW + lane / NP;
    const int c = cbase + cl;
    const bool cvalid = c < cend;
    const bool lvalid = cvalid && n < N;
    const int cc = cvalid ? c : cend - 1, nn = n < N ? n : N - 1;

    const float A2 = lvalid ? p.A[(int64_t)cc * p.A_d_stride + (int64_t)nn * p.A_dstate_stride] * kLog2e : 0.f;
    const float ld = p.A_decay ? __log2f(p.A_decay[0]) : 0.f;

    const T *Bp = (const T *)p.B + (int64_t)b * p.B_batch_stride + (int64_t)g * p.B_group_stride;
    const T *Cp = (const T *)p.C + (int64_t)b * p.C_batch_stride + (int64_t)g * p.C_group_stride;
    const T *up = (const T *)p.u + (int64_t)b * p.u_batch_stride;
    const T *dp = (const T *)p.delta + (int64_t)b * p.delta_batch_stride;
    TO *op = (TO *)p.out + (int64_t)b * p.out_batch_stride;

    const int64_t plane = ((int64_t)b * Dm + cc) * N + nn;
    float *xv = p.x_v + plane * geo.nCY * geo.Wp;
    float *xh = SAVE ? p.x + plane * geo.nCX * geo.Hp : nullptr;
    float *xs = SAVE ? p.x_sd + plane * geo.nCX * geo.Hp : nullptr;

    const int nJ = (W + TC - 1) / TC;
    const float *myDl = sDl + cl * (R + 1) * TC;
    const float *myDu = sDu + cl * R * TC;
    const float *myB = sB + n * NSTR;
    const float *myC = sC + n * NSTR;

    for (int I = 0; I < geo.nCY; ++I) {
        const int r0 = I * R;
        const int rn = min(R, H - r0);
        float hl[R], sl[R], al[R];                  // h, s, a at the column left of the tile
#pragma unroll
        for (int r = 0; r < R; ++r) { hl[r] = 0.f; sl[r] = 0.f; al[r] = 0.f; }

        for (int J = 0; J < nJ; ++J) {
            const int j0 = J * TC;
            const int tcn = min(TC, W - j0);

            // ---- stage B, C (all states, this tile) : zero outside the plane and for n >= N
            for (int idx = tid; idx < NP * R * TC; idx += kThreads) {
                const int sn = idx / (R * TC), rem = idx - sn * (R * TC);
                const int r = rem / TC, j = rem - r * TC;
                float vb = 0.f, vc = 0.f;
                if (sn < N && r < rn && j < tcn) {
                    const int64_t off = (int64_t)(r0 + r) * p.B_h_stride + (j0 + j);
                    vb = to_f32(Bp[(int64_t)sn * p.B_dstate_stride + off]);
                    const int64_t offc = (int64_t)(r0 + r) * p.C_h_stride + (j0 + j);
                    vc = to_f32(Cp[(int64_t)sn * p.C_dstate_stride + offc]);
                }
                sB[sn * NSTR + rem] = vb;
                sC[sn * NSTR + rem] = vc;
            }
            // ---- stage delta' (rows r0-1 .. r0+R-1) and delta'*u : once per pixel, not per state
            for (int idx = tid; idx < CB * (R + 1) * TC; idx += kThreads) {
                const int scl = idx / ((R + 1) * TC), rem = idx - scl * ((R + 1) * TC);
                const int rr = rem / TC, j = rem - rr * TC;
                const int sc = cbase + scl, row = r0 - 1 + rr, col = j0 + j;
                float dl = 0.f, du = 0.f;
                if (sc < cend && row >= 0 && row < H && col < W) {
                    const int dgi = sc / rd;
                    float raw = to_f32(dp[(int64_t)dgi * p.delta_d_stride + (int64_t)row * p.delta_h_stride + col]);
                    if (p.delta_bias) raw += p.delta_bias[dgi];
                    dl = p.delta_softplus ? softplus20(raw) : raw;
                    if (rr > 0) du = dl * to_f32(up[(int64_t)sc * p.u_d_stride + (int64_t)row * p.u_h_stride + col]);
                }
                sDl[idx] = dl;
                if (rr > 0) sDu[scl * R * TC + (rr - 1) * TC + j] = du;
            }
            __syncthreads();

            // ---- per-lane tile walk
            float hup[TC], aup[TC];                 // row above the current one
            float corner = 0.f;                     // h[r0-1][j0-1]
            if (I > 0) {
                const float4 *src = (const float4 *)(xv + (int64_t)(I - 1) * geo.Wp + j0);
#pragma unroll
                for (int k = 0; k < TC / 4; ++k) {
                    const float4 v = src[k];
                    hup[4 * k + 0] = v.x; hup[4 * k + 1] = v.y; hup[4 * k + 2] = v.z; hup[4 * k + 3] = v.w;
                }
#pragma unroll
                for (int j = 0; j < TC; ++j) {
                    hup[j] = lvalid ? hup[j] : 0.f;
                    aup[j] = fast_exp2(fmaf(myDl[j], A2, ld));
                }
                if (J > 0) corner = lvalid ? xv[(int64_t)(I - 1) * geo.Wp + j0 - 1] : 0.f;
            } else {
#pragma unroll
                for (int j = 0; j < TC; ++j) { hup[j] = 0.f; aup[j] = 0.f; }
            }

            float xe[NG][R], xse[NG][R];            // h, s at checkpoint columns
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r < rn) {
                    float left = hl[r], sleft = sl[r], aleft = al[r];
                    float diag = corner;
                    corner = hl[r];                 // h[r0+r][j0-1] is the next row's corner
                    float y[TC];
#pragma unroll
                    for (int j4 = 0; j4 < TC; j4 += 4) {
                        const float4 vdl = *(const float4 *)(myDl + (r + 1) * TC + j4);
                        const float4 vdu = *(const float4 *)(myDu + r * TC + j4);
                        const float4 vb = *(const float4 *)(myB + r * TC + j4);
                        const float4 vc = *(const float4 *)(myC + r * TC + j4);
                        const float adl[4] = {vdl.x, vdl.y, vdl.z, vdl.w};
                        const float adu[4] = {vdu.x, vdu.y, vdu.z, vdu.w};
                        const float ab[4] = {vb.x, vb.y, vb.z, vb.w};
                        const float ac[4] = {vc.x, vc.y, vc.z, vc.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int j = j4 + q;
                            if (j < tcn) {
                                const float a = fast_exp2(fmaf(adl[q], A2, ld));
                                const float bu = ab[q] * adu[q];
                                const float X = fmaf(-0.5f * (aup[j] + aleft), diag, hup[j]);
                                const float h = fmaf(a, left + X, bu);
                                const float s = fmaf(a, sleft, bu);
                                y[j] = ac[q] * fmaf(0.25f, bu, h - s);
                                diag = hup[j];
                                hup[j] = h; aup[j] = a;
                                left = h; aleft = a; sleft = s;
                                if ((j & (kCkX - 1)) == kCkX - 1) { xe[j / kCkX][r] = h; xse[j / kCkX][r] = s; }
                            } else {
                                y[j] = 0.f;
                            }
                        }
                    }
                    hl[r] = left; sl[r] = sleft; al[r] = aleft;
#pragma unroll
                    for (int j = 0; j < TC; ++j) y[j] = group_sum<NP>(y[j]);
                    if (n == 0) {
                        float4 *dst = (float4 *)(sY + cl * R * TC + r * TC);
#pragma unroll
                        for (int k = 0; k < TC / 4; ++k) dst[k] = make_float4(y[4 * k], y[4 * k + 1], y[4 * k + 2], y[4 * k + 3]);
                    }
                } else {
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi) { xe[gi][r] = 0.f; xse[gi][r] = 0.f; }
                }
            }
            if (lvalid) {
                // row checkpoint / carry to the next strip: h at the strip's last row
                float4 *dst = (float4 *)(xv + (int64_t)I * geo.Wp + j0);
#pragma unroll
                for (int k = 0; k < TC / 4; ++k) dst[k] = make_float4(hup[4 * k], hup[4 * k + 1], hup[4 * k + 2], hup[4 * k + 3]);
                if (SAVE) {
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi) {
                        if (gi * kCkX + kCkX <= tcn) {
                            const int Jb = (j0 + gi * kCkX) / kCkX;
                            float4 *dh = (float4 *)(xh + (int64_t)Jb * geo.Hp + r0);
                            float4 *ds = (float4 *)(xs + (int64_t)Jb * geo.Hp + r0);
#pragma unroll
                            for (int k = 0; k < R / 4; ++k) {
                                dh[k] = make_float4(xe[gi][4 * k], xe[gi][4 * k + 1], xe[gi][4 * k + 2], xe[gi][4 * k + 3]);
                                ds[k] = make_float4(xse[gi][4 * k], xse[gi][4 * k + 1], xse[gi][4 * k + 2], xse[gi][4 * k + 3]);
                            }
                        }
                    }
                }
            }
            __syncthreads();

            // ---- out = D*u + y, written by the whole block, coalesced along the row
            for (int idx = tid; idx < CB * R * TC; idx += kThreads) {
                const int scl = idx / (R * TC), rem = idx - scl * (R * TC);
                const int r = rem / TC, j = rem - r * TC;
                const int sc = cbase + scl;
                if (sc < cend && r < rn && j < tcn) {
                    const int row = r0 + r, col = j0 + j;
                    float v = sY[idx];
                    if (p.D) v = fmaf(p.D[sc], to_f32(up[(int64_t)sc * p.u_d_stride + (int64_t)row * p.u_h_stride + col]), v);
                    op[(int64_t)sc * p.out_d_stride + (int64_t)row * p.out_h_stride + col] = from_f32<TO>(v);
                }
            }
            // the next tile's staging does not touch sY, and its first barrier orders the
            // sY reads above against the next tile's sY writes
        }
    }
}

template <typename T, typename TO, int NP>
static int launch_fwd_np(const snd_fwd_params &p, hipStream_t stream) {
    constexpr int TC = 8;
    // waves per block: keep channels per block (and with it the per-channel LDS tiles) bounded
    constexpr int WPB = NP >= 8 ? 4 : (NP == 4 ? 2 : 1);
    constexpr int CB = (kWave / NP) * WPB;
    constexpr int kThreads = WPB * kWave;
    const snd_shape &sh = p.shape;
    const Geo geo = make_geo(sh.nrows, sh.ncols);
    const int rg = sh.dim / sh.n_groups;
    const int nChunks = (rg + CB - 1) / CB;
    const int grid = xcd_grid(sh.batch * sh.n_groups, nChunks);
    const bool save = p.x != nullptr;
    if (save)
        hipLaunchKernelGGL((fwd_kernel<T, TO, NP, WPB, TC, true>), dim3(grid), dim3(kThreads), 0, stream, p, geo);
    else
        hipLaunchKernelGGL((fwd_kernel<T, TO, NP, WPB, TC, false>), dim3(grid), dim3(kThreads), 0, stream, p, geo);
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T, typename TO>
static int launch_fwd_t(const snd_fwd_params &p, hipStream_t stream) {
    const int N = p.shape.dstate;
    if (N > 8) return launch_fwd_np<T, TO, 16>(p, stream);
    if (N > 4) return launch_fwd_np<T, TO, 8>(p, stream);
    if (N > 2) return launch_fwd_np<T, TO, 4>(p, stream);
    if (N > 1) return launch_fwd_np<T, TO, 2>(p, stream);
    return launch_fwd_np<T, TO, 1>(p, stream);
}

int launch_fwd(const snd_fwd_params &p, hipStream_t stream) {
    const int it = p.shape.in_dtype, ot = p.out_dtype;
    if (it == SND_F32 && ot == SND_F32) return launch_fwd_t<float, float>(p, stream);
    if (it == SND_BF16 && ot == SND_F32) return launch_fwd_t<bf16_t, float>(p, stream);
    if (it == SND_BF16 && ot == SND_BF16) return launch_fwd_t<bf16_t, bf16_t>(p, stream);
    if (it == SND_F16 && ot == SND_F32) return launch_fwd_t<f16_t, float>(p, stream);
    if (it == SND_F16 && ot == SND_F16) return launch_fwd_t<f16_t, f16_t>(p, stream);
    return SND_ERR_DTYPE;
}

}  // namespace snd
