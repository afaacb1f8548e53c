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
// the columns.  Every load, store and the whole adjoint sweep therefore use the mirrored order (lane l =
// column 64w + 63 - l); only the recomputation of h and s, which runs with the columns, sees its inputs and
// leaves its results through a lane reversal (ds_bpermute: a register crossbar move, no LDS memory).
// A wave handles its segment band by band (R rows), bottom band first: recompute h, s of the band's rows
// from the forward's checkpoints (row above the band from x_v, what entered the segment on every row from
// x / x_sd: no wave waits for another here), then sweep the band's rows bottom-up.  The sweep needs G, Gs, a
// of the segment on the right at its first column: wave w runs one band behind wave w+1 and finds them in
// LDS (one block barrier per band, no polling).  dB, dC leave as one global atomic per element and channel
// (a wave-wide instruction covers 256 consecutive bytes), du / ddelta as whole row segments.
#pragma once
#include <type_traits>
#include "snd_device.h"

namespace snd {

__device__ __forceinline__ void wave_glb_add(float *p, float v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, int NS, bool DO32>
__global__ __launch_bounds__(64 * kMaxSeg) void wave_bwd_kernel(const snd_bwd_params p, const WaveGeo wg) {
    constexpr int R = NS <= 1 ? 8 : 4;               // rows per band
    constexpr bool PF = NS <= 2;                     // load a band's inputs one band ahead (with four states the registers are needed elsewhere)
    // what a wave leaves for the wave on its left: {G, Gs, a, -} at its first column, per band parity, row and
    // state.  Wave w writes slot w and reads slot w+1; the slot after the last wave stays zero.
    __shared__ float4 sHO[2][kMaxSeg + 1][R][NS];

    const snd_fwd_params &f = p.f;
    const snd_shape &sh = f.shape;
    const int H = sh.nrows, W = sh.ncols, N = sh.dstate, Dm = sh.dim, G = sh.n_groups;
    const int rg = Dm / G, rd = Dm / sh.delta_dim;
    int pair, chunk;
    if (!wave_job(blockIdx.x, sh.batch * G, rg, pair, chunk)) return;
    const int b = pair / G, g = pair - b * G, c = g * rg + chunk;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int nseg = wg.nseg;
    const bool multi = nseg > 1;
    if (threadIdx.x < 2 * R * NS) (&sHO[0][0][0][0])[((threadIdx.x / (R * NS)) * (kMaxSeg + 1) + nseg) * R * NS + threadIdx.x % (R * NS)] = make_float4(0.f, 0.f, 0.f, 0.f);

    const bool fv = f.directions == SND_DIR_CORNERS && (g & 2), fh = f.directions == SND_DIR_CORNERS && (g & 1);
    const int r0m = fv ? H - 1 : 0, rs = fv ? -1 : 1;
    const int jm = w * kSeg + 63 - lane;             // this lane's column (mirrored order)
    const bool jin = jm < W;
    const int jc = jin ? jm : W - 1;
    const int mc = fh ? W - 1 - jc : jc;
    const int jn = w * kSeg + lane;                  // natural order (row checkpoints, recomputation)
    const int rev_addr = (63 - lane) * 4;
    auto mirror = [&](float v) {
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(rev_addr, __builtin_bit_cast(int, v)));
    };
    auto bcast = [](float v, int src_lane) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src_lane));
    };

    float Av[NS], A2[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        Av[n] = n < N ? f.A[(int64_t)c * f.A_d_stride + (int64_t)n * f.A_dstate_stride] : 0.f;
        A2[n] = Av[n] * kLog2e;
    }
    const float ld = f.A_decay ? __log2f(f.A_decay[0]) : 0.f;
    const float Dv = f.D ? f.D[c] : 0.f;
    const float bias = f.delta_bias ? f.delta_bias[c / rd] : 0.f;
    const bool softplus = f.delta_softplus != 0;
    const bool want_decay = p.dA_decay != nullptr;

    constexpr int ESZ = (int)sizeof(T);
    using DoT = typename std::conditional<DO32, float, T>::type;
    constexpr int DSZ = (int)sizeof(DoT);
    const T *Bb = (const T *)f.B + (int64_t)b * f.B_batch_stride + (int64_t)g * f.B_group_stride;
    const T *Cb = (const T *)f.C + (int64_t)b * f.C_batch_stride + (int64_t)g * f.C_group_stride;
    const T *ub = (const T *)f.u + (int64_t)b * f.u_batch_stride + (int64_t)(f.u_shared ? chunk : c) * f.u_d_stride;
    const T *db = (const T *)f.delta + (int64_t)b * f.delta_batch_stride + (int64_t)(c / rd) * f.delta_d_stride;
    const DoT *dob = (const DoT *)p.dout + (int64_t)b * p.dout_batch_stride + (int64_t)c * p.dout_d_stride;
    T *dub = (T *)p.du + ((int64_t)b * Dm + c) * H * W;                 // du, ddelta: dense [b, c, H, W]
    T *ddb = (T *)p.ddelta + ((int64_t)b * Dm + c) * H * W;
    float *dBg = p.dB + ((int64_t)b * G + g) * N * H * W;               // dense [b, g, N, H, W]
    float *dCg = p.dC + ((int64_t)b * G + g) * N * H * W;
    // byte steps from one scan row to the next (negative when the group scans bottom-up) and column offsets
    const int UhB = (int)f.u_h_stride * ESZ * rs, DhB = (int)f.delta_h_stride * ESZ * rs, BhB = (int)f.B_h_stride * ESZ * rs,
              ChB = (int)f.C_h_stride * ESZ * rs, DohB = (int)p.dout_h_stride * DSZ * rs, WB = W * ESZ * rs, W4 = W * 4 * rs;
    const int64_t BsB = f.B_dstate_stride * ESZ, CsB = f.C_dstate_stride * ESZ, HW4 = (int64_t)H * W * 4;
    const uint32_t colB = (uint32_t)mc * ESZ, colO = (uint32_t)mc * DSZ, col4 = (uint32_t)mc * 4;

    // saved state of this plane set (layouts in snd_device.h)
    const int64_t plane0 = ((int64_t)b * Dm + c) * N;
    const float *xv = f.x_v + plane0 * wave_xv_plane(wg) + jn;
    const float *xh = f.x + plane0 * wave_x_plane(wg) + (int64_t)w * 2 * wg.Hp;
    const float *xs = f.x_sd + plane0 * wave_x_plane(wg) + (int64_t)w * 2 * wg.Hp;

    // Inputs of one band.  Rows wait as raw bits in mirrored lane order; lanes beyond the last column read the
    // last column (always in bounds) and only their dout is masked to zero where it is used, which makes every
    // adjoint there exactly zero.  h0, a0: the row above the band in natural order.  ch, cs, ca: what entered
    // the segment from the left on rows i0-1 .. i0+R-1, one row per lane.
    struct In { uint32_t u[R], d[R], o[R], b[R][NS], c[R][NS]; float h0[NS], a0[NS], ch[NS], cs[NS], ca[NS]; };
    const T *const tp = nullptr;                     // selects the conversions
    const DoT *const dp = nullptr;
    // Every band issues the same loads on every path (the wait counters the compiler derives for the prefetch
    // need that): rows past the end of a ragged last band read the last row again and are never used.
    auto load_band = [&](In &q, int band) {
        const int i0 = band * R;
        const int m0 = mad24(i0, rs, r0m);           // memory row of the band's first scan row
        uint32_t ou = mad24(m0, UhB * rs, colB), od = mad24(m0, DhB * rs, colB), oo = mad24(m0, DohB * rs, colO),
                 ob = mad24(m0, BhB * rs, colB), oc = mad24(m0, ChB * rs, colB);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            q.u[r] = ldraw_b(ub, ou);
            q.d[r] = ldraw_b(db, od);
            q.o[r] = ldraw_b(dob, oo);
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                const int sn = (NS == 4 && n >= N) ? 0 : n;
                q.b[r][n] = ldraw_b((const T *)((const char *)Bb + sn * BsB), ob);
                q.c[r][n] = ldraw_b((const T *)((const char *)Cb + sn * CsB), oc);
            }
            const bool more = i0 + r + 1 < H;
            ou += more ? UhB : 0; od += more ? DhB : 0; oo += more ? DohB : 0; ob += more ? BhB : 0; oc += more ? ChB : 0;
        }
        const int row = i0 - 1 + lane;
#pragma unroll
        for (int n = 0; n < NS; ++n) {
            q.h0[n] = 0.f; q.a0[n] = 0.f; q.ch[n] = 0.f; q.cs[n] = 0.f; q.ca[n] = 0.f;
            if (NS != 4 || n < N) {
                if (band > 0) {
                    const float *src = xv + (int64_t)n * wave_xv_plane(wg) + (int64_t)(band - 1) * 2 * wg.Wp;
                    q.h0[n] = __builtin_nontemporal_load(src);
                    q.a0[n] = __builtin_nontemporal_load(src + wg.Wp);
                }
                if (w > 0 && lane <= R && row >= 0) {
                    const int64_t o = (int64_t)n * wave_x_plane(wg) + row;
                    q.ch[n] = xh[o];
                    q.ca[n] = xh[o + wg.Hp];
                    q.cs[n] = xs[o];
                }
            }
        }
    };

    float Gd[NS], ad[NS], GdEdge[NS];               // G, a of the row below at this column; G[i+1, 64(w+1)]
    float dA_acc[NS];
    float dec_acc = 0.f, dD_acc = 0.f, dbias_acc = 0.f;
#pragma unroll
    for (int n = 0; n < NS; ++n) { Gd[n] = 0.f; ad[n] = 0.f; GdEdge[n] = 0.f; dA_acc[n] = 0.f; }
    int step = nseg - 1 - w;                         // the waves on the right go first
    const bool hands_over = multi && w > 0;

    // one band from `cur`, with the loads of the band above issued into `nxt` first
    auto do_band = [&](In &cur, In &nxt, int band) {
        if (PF) { if (band > 0) load_band(nxt, band - 1); }
        else load_band(cur, band);
        const int i0 = band * R;

        // ---- recompute h, s on the band's rows (with the columns); results back in mirrored order
        float hT[R][NS], sT[R][NS], aT[R][NS], dl[R], dsp[R], hTop[NS];
        {
            float hp[NS], ap[NS], hdiag[NS];
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                hp[n] = cur.h0[n];
                ap[n] = cur.a0[n];
                hdiag[n] = bcast(cur.ch[n], 0);
                hTop[n] = mirror(cur.h0[n]);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                dl[r] = 0.f;
                dsp[r] = 0.f;
                if (i0 + r < H) {
                    const float raw = cvt_raw(tp, cur.d[r]) + bias;
                    float sg = 1.f;
                    dl[r] = softplus ? softplus20(raw, sg) : raw;
                    dsp[r] = sg;
                    const float dl_n = mirror(dl[r]), dlu_n = mirror(dl[r] * cvt_raw(tp, cur.u[r]));
#pragma unroll
                    for (int n = 0; n < NS; ++n) {
                        const float hin = bcast(cur.ch[n], r + 1), sin_ = bcast(cur.cs[n], r + 1), ain = bcast(cur.ca[n], r + 1);
                        const float a = fast_exp2(fmaf(dl_n, A2[n], ld));
                        const float bu = ((NS == 4 && n >= N) ? 0.f : mirror(cvt_raw(tp, cur.b[r][n]))) * dlu_n;
                        const float a_l = from_prev_lane(a, ain);              // a[i, j-1]
                        const float h_d = from_prev_lane(hp[n], hdiag[n]);     // h[i-1, j-1]
                        const float X = fmaf(-0.5f * (ap[n] + a_l), h_d, hp[n]);
                        float Y = fmaf(a, X, bu), S = bu, Ap = a;
                        wave_scan3(Y, S, Ap);
                        const float h = fmaf(Ap, hin, Y);
                        const float s = fmaf(Ap, sin_, S);
                        hT[r][n] = mirror(h);
                        sT[r][n] = mirror(s);
                        aT[r][n] = mirror(a);
                        hp[n] = h;
                        ap[n] = a;
                        hdiag[n] = hin;
                    }
                } else {
#pragma unroll
                    for (int n = 0; n < NS; ++n) { hT[r][n] = 0.f; sT[r][n] = 0.f; aT[r][n] = 0.f; }
                }
            }
        }

        // ---- adjoint sweep over the band's rows, bottom-up (against the columns)
        const int rows = min(R, H - i0);             // rows of this band inside the plane
        const int mlast = mad24(i0 + rows - 1, rs, r0m);
        uint32_t og = mad24(mlast, WB * rs, colB), o4 = mad24(mlast, W4 * rs, col4);   // du / ddelta and dB / dC offsets of the row
#pragma unroll
        for (int r = R - 1; r >= 0; --r) {
            if (i0 + r < H) {
                const float dov = jin ? cvt_raw(dp, cur.o[r]) : 0.f, uv = cvt_raw(tp, cur.u[r]), dlv = dl[r];
                const float dlu = dlv * uv;
                float qsum = 0.f, psum = 0.f;
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    // what the segment on the right left for this row: G, Gs, a at column 64(w+1)
                    const float4 in = sHO[(step + 1) & 1][w + 1][r][n];
                    const float hin = bcast(cur.ch[n], r + 1);                 // h[i, 64w-1]
                    const bool live = NS != 4 || n < N;
                    const float Bv = live ? cvt_raw(tp, cur.b[r][n]) : 0.f, Cv = live ? cvt_raw(tp, cur.c[r][n]) : 0.f;
                    const float a = aT[r][n];
                    const float bu = Bv * dlu;
                    const float dyC = dov * Cv;
                    const float a_r = from_prev_lane(a, in.z);                 // a[i, j+1]
                    const float Gdiag = from_prev_lane(Gd[n], GdEdge[n]);      // G[i+1, j+1]
                    const float z = fmaf(-0.5f * (a_r + ad[n]), Gdiag, dyC + Gd[n]);
                    float Y = a * z, S = -a * dyC, Ap = a;
                    wave_scan3(Y, S, Ap);
                    const float Gt = fmaf(Ap, in.x, Y), Gst = fmaf(Ap, in.y, S);   // G[i,j], Gs[i,j]
                    const float Gr = from_prev_lane(Gt, in.x), Gsr = from_prev_lane(Gst, in.y);
                    const float g_ = Gr + z, gs = Gsr - dyC;
                    const float dbu = fmaf(0.25f, dyC, g_ + gs);
                    const float hv = hT[r][n], sv = sT[r][n];
                    const float h_l = from_next_lane(hv, hin);                 // h[i, j-1]
                    const float h_u = r > 0 ? hT[r > 0 ? r - 1 : 0][n] : hTop[n];
                    const float hs = hv - sv, sb = sv - bu;
                    const float cross = fmaf(Gd[n], h_l, Gr * h_u);
                    const float da = fmaf(-0.5f * a, cross, fmaf(g_, hs, (g_ + gs) * sb));
                    dA_acc[n] = fmaf(dlv, da, dA_acc[n]);
                    if (want_decay) dec_acc += da;
                    qsum = fmaf(dbu, Bv, qsum);
                    psum = fmaf(Av[n], da, psum);
                    if (jin && live) {
                        wave_glb_add((float *)((char *)dBg + n * HW4 + o4), dbu * dlu);
                        wave_glb_add((float *)((char *)dCg + n * HW4 + o4), dov * fmaf(0.25f, bu, hs));
                    }
                    GdEdge[n] = in.x;
                    Gd[n] = Gt;
                    ad[n] = a;
                    if (hands_over && lane == 63) sHO[step & 1][w][r][n] = make_float4(Gt, Gst, a, 0.f);
                }
                const float duv = fmaf(Dv, dov, dlv * qsum);
                const float ddl = fmaf(uv, qsum, psum) * dsp[r];
                if (jin) {
                    dD_acc = fmaf(dov, uv, dD_acc);
                    dbias_acc += ddl;
                    stg_b(dub, og, duv);
                    stg_b(ddb, og, ddl);
                }
                og -= WB;
                o4 -= W4;
            }
        }
        if (multi) { lds_barrier(); ++step; }
    };

    In sA;
    if (PF) load_band(sA, wg.nBands - 1);
    lds_barrier();                                   // the zeroed slot
    if (multi)
        for (int e = 0; e < nseg - 1 - w; ++e) lds_barrier();
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
        for (int e = 0; e < w; ++e) lds_barrier();

    // ---- per-channel sums leave the kernel: one atomic per wave and value
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        const float t = wave_sum_to_last(dA_acc[n]);
        if (lane == 63 && n < N) wave_glb_add(p.dA + (int64_t)c * N + n, t);
    }
    {
        const float td = wave_sum_to_last(dD_acc), tb = wave_sum_to_last(dbias_acc);
        if (lane == 63) {
            if (p.dD) wave_glb_add(p.dD + c, td);
            if (p.ddelta_bias) wave_glb_add(p.ddelta_bias + c, tb);
        }
    }
    if (want_decay) {
        const float t = wave_sum_to_last(dec_acc);
        if (lane == 63) wave_glb_add(p.dA_decay, t / f.A_decay[0]);
    }
}

template <typename T, int NS>
static int launch_wave_bwd_ns(const snd_bwd_params &p, hipStream_t stream) {
    const snd_shape &sh = p.f.shape;
    const WaveGeo wg = make_wave_geo(sh.nrows, sh.ncols, sh.dstate);
    const dim3 grid(wave_grid(sh.batch * sh.n_groups, sh.dim / sh.n_groups)), block(64 * wg.nseg);
    if (p.dout_dtype == SND_F32) hipLaunchKernelGGL((wave_bwd_kernel<T, NS, true>), grid, block, 0, stream, p, wg);
    else hipLaunchKernelGGL((wave_bwd_kernel<T, NS, std::is_same<T, float>::value>), grid, block, 0, stream, p, wg);
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

template <typename T>
int launch_wave_bwd_t(const snd_bwd_params &p, hipStream_t stream) {
    const int N = p.f.shape.dstate;
    return N == 1 ? launch_wave_bwd_ns<T, 1>(p, stream) : N == 2 ? launch_wave_bwd_ns<T, 2>(p, stream)
                                                                  : launch_wave_bwd_ns<T, 4>(p, stream);
}

}  // namespace snd
