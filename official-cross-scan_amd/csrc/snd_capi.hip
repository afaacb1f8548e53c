// C ABI of the gfx950 selective_nd_scan library: validation, planning and dispatch.
// Mirrors the checks of the reference host binding
// (kernels/selective_nd_scan/src/cusoflex/selective_scan_oflex.cpp:188-245,298-361) as status codes.
#include <algorithm>
#include <atomic>
#include <functional>
#include <map>
#include <mutex>
#include <queue>
#include <tuple>
#include <vector>

#include "snd_device.h"

namespace snd {
int launch_fwd_f32(const snd_fwd_params &p, hipStream_t stream);
int launch_fwd_bf16(const snd_fwd_params &p, hipStream_t stream);
int launch_fwd_f16(const snd_fwd_params &p, hipStream_t stream);
int launch_bwd_f32(const snd_bwd_params &p, hipStream_t stream);
int launch_bwd_bf16(const snd_bwd_params &p, hipStream_t stream);
int launch_bwd_f16(const snd_bwd_params &p, hipStream_t stream);
int launch_wave_fwd_f32(const snd_fwd_params &p, float *group_ws, hipStream_t stream);
int launch_wave_fwd_bf16(const snd_fwd_params &p, float *group_ws, hipStream_t stream);
int launch_wave_fwd_f16(const snd_fwd_params &p, float *group_ws, hipStream_t stream);
int launch_wave_bwd_f32(const snd_bwd_params &p, float *group_ws, hipStream_t stream);
int launch_wave_bwd_bf16(const snd_bwd_params &p, float *group_ws, hipStream_t stream);
int launch_wave_bwd_f16(const snd_bwd_params &p, float *group_ws, hipStream_t stream);
int configure_bwd_f32();
int configure_bwd_bf16();
int configure_bwd_f16();
}  // namespace snd

// Scratch of snd_bwd_static(): one array per GPU the library runs on, held until the process ends.
// Host code never uses the array's name as an address: ensure_device_ready() asks the runtime for the
// array's device address on each GPU and every later use goes through that pointer.
#define SND_STATIC_WORKSPACE_BYTES (64ll << 20)
static __device__ __align__(256) unsigned char scratch[SND_STATIC_WORKSPACE_BYTES];

namespace snd {
__global__ void zero_words_kernel(int *p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}
int zero_words(int *p, int64_t n, hipStream_t stream) {
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, n);
    return hipGetLastError() == hipSuccess ? SND_OK : SND_ERR_LAUNCH;
}

constexpr int kMaxDevices = 64;
static std::mutex g_setup_mutex;
static std::atomic<bool> g_ready[kMaxDevices];
static void *g_scratch[kMaxDevices];                // device address of `scratch` on each GPU
static std::atomic<int> g_spin_limit{kSpinLimit};

int spin_limit() { return g_spin_limit.load(std::memory_order_relaxed); }

// Tile steps the strip pipeline takes: jobs (plane chunk, strip, segment) in ticket order, each taken by the first
// free slot; a tile starts when its block has finished the tile before it, the same tile of the strip before it is
// done and, for a segment's first tile, the segment before it is done.
static double strip_pipeline_steps(int nPC, int nS, int nT, int slots, int nSeg) {
    const int L = nT / nSeg;
    std::vector<double> fin((size_t)nPC * nS * nT, 0.0);           // finish time of every tile
    std::priority_queue<double, std::vector<double>, std::greater<double>> free;
    for (int i = 0; i < slots; ++i) free.push(0.0);
    double end = 0.0;
    for (int key = 0; key < nS + (nSeg - 1) * L; ++key)
        for (int g = 0; g < nSeg; ++g) {
            const int s_ = key - g * L;
            if (s_ < 0 || s_ >= nS) continue;
            const int j0 = g * L, j1 = g == nSeg - 1 ? nT : j0 + L;
            for (int pc = 0; pc < nPC; ++pc) {
                double t = free.top();
                free.pop();
                double *row = &fin[((size_t)pc * nS + s_) * nT];
                const double *prev = s_ > 0 ? row - nT : nullptr;
                if (g > 0 && row[j0 - 1] > t) t = row[j0 - 1];
                for (int j = j0; j < j1; ++j) {
                    if (prev && prev[j] > t) t = prev[j];
                    t += 1.0;
                    row[j] = t;
                }
                free.push(t);
                if (t > end) end = t;
            }
        }
    return end;
}
static std::atomic<int> g_strip_slots{0};           // test hook: block slots the model assumes (0: the machine's)
int strip_segments(int64_t nPlaneChunks, int nStrips, int nTilesX, int64_t slots, int nQueues) {
    if (const int forced = g_strip_slots.load(std::memory_order_relaxed)) {
        if (forced < 0) return nQueues == 1 && nStrips >= 2 ? std::max(1, std::min(-forced, nTilesX / 2)) : 1;   // that many segments
        slots = forced;
    }
    if (nQueues != 1 || nStrips < 2 || nTilesX < 8 || nPlaneChunks * nStrips <= slots ||
        nPlaneChunks * nStrips * nTilesX > ((int64_t)1 << 21))
        return 1;
    static std::mutex m;
    static std::map<std::tuple<int64_t, int, int, int64_t>, int> cache;
    const auto key = std::make_tuple(nPlaneChunks, nStrips, nTilesX, slots);
    std::lock_guard<std::mutex> lock(m);
    const auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    int best = 1;
    const double whole = strip_pipeline_steps((int)nPlaneChunks, nStrips, nTilesX, (int)slots, 1);
    double best_cost = whole;
    for (int nSeg = 2; nSeg <= 4 && nTilesX / nSeg >= 4; ++nSeg) {
        const double cost = strip_pipeline_steps((int)nPlaneChunks, nStrips, nTilesX, (int)slots, nSeg) * (1.0 + 0.02 * (nSeg - 1));
        if (cost < best_cost && cost < whole * 0.92) { best = nSeg; best_cost = cost; }
    }
    cache[key] = best;
    return best;
}

// Set-up of the current device: done once, by whichever of snd_init() and the first launch comes first.
int ensure_device_ready() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SND_ERR_LAUNCH;
    if (g_ready[dev].load(std::memory_order_acquire)) return SND_OK;
    std::lock_guard<std::mutex> lock(g_setup_mutex);
    if (g_ready[dev].load(std::memory_order_relaxed)) return SND_OK;
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return SND_ERR_LAUNCH;
    g_scratch[dev] = ptr;
    if (configure_bwd_f32() != SND_OK || configure_bwd_bf16() != SND_OK || configure_bwd_f16() != SND_OK) return SND_ERR_LAUNCH;
    g_ready[dev].store(true, std::memory_order_release);
    return SND_OK;
}
static void *device_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    return g_ready[dev].load(std::memory_order_acquire) ? g_scratch[dev] : nullptr;
}
}  // namespace snd

namespace {

int64_t plane_chunks(const snd_shape &s) {
    return (int64_t)s.batch * s.n_groups * ((s.dim / s.n_groups + 15) / 16);
}

// Where the column groups of a wide plane (row-segment kernels) hand over inside a workspace: behind the sync words
int64_t group_ws_offset(const snd_shape &s) {
    const snd::Geo g = snd::make_geo(s.nrows, s.ncols);
    return (snd::sync_words(plane_chunks(s), g.nCY) * (int64_t)sizeof(int) + 255) / 256 * 256;
}

int check_shape(const snd_shape &s) {
    if (s.batch <= 0 || s.dim <= 0 || s.nrows <= 0 || s.ncols <= 0 || s.dstate <= 0 || s.n_groups <= 0 ||
        s.delta_dim <= 0)
        return SND_ERR_SHAPE;
    if (s.dim % s.n_groups != 0) return SND_ERR_SHAPE;      // host.cpp:215
    if (s.dim % s.delta_dim != 0) return SND_ERR_SHAPE;     // host.cpp:216
    if (s.dstate > SND_MAX_DSTATE) return SND_ERR_SHAPE;    // host.cpp:217
    if (s.in_dtype != SND_F32 && s.in_dtype != SND_F16 && s.in_dtype != SND_BF16) return SND_ERR_DTYPE;
    return SND_OK;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// Which of the two kernel families is the faster one for a shape with 1-4 states, from a model of the backward
// (the longer kernel) fitted to measurements on one MI355X (32 x D x HxW planes, D*H*W constant, H = W = 7 .. 112,
// N = 1, 2, 4, bf16):
//   * row-segment wavefront: a plane is a block of nseg waves, 2048 waves fit the chip at once, a wave takes a
//     row of its segment in about 0.85 us (one state), 1.5 (two), 2.95 (three or four), whatever the row's width.
//     Where four channels share their dB / dC atomics (one segment per plane, 512 planes or more) a row takes 0.7,
//     1.15, 2.4 us.  Planes of at most 32 / 16 columns are packed two / four to a wave, whose row then takes 0.65,
//     1.05, 2.05 us; planes of at most 7 columns eight to a wave, 0.75, 1.15, 2.2 us.
//   * tile kernels with four lanes per channel: a block is one wave of 16 channels, 1024 fit at once, and a block
//     takes one 8x8 (7x7) tile in about 18.5 us - or, with few blocks and many strips, the strip pipeline takes
//     (column tiles + strips - 1) steps of about 25 us per round of its jobs.
// With four states, planes of 33 to 40 columns go to the tile kernels (32 x 384 x 40x40: 0.65 ms forward + backward
// instead of 0.73), everything else to the wavefront (32 x 12288 x 7x7, four states: 0.59 ms instead of 0.65; 32 x 3072
// x 14x14, one state: 0.18 instead of 0.60; 32 x 192 x 56x56, one state: 0.18 instead of 0.67; 512x512 x 256 channels,
// one state: 0.65 instead of 3.2).
bool wave_family_pays(const snd_shape &s) {
    const snd::Geo g = snd::make_geo(s.nrows, s.ncols);
    const snd::WaveGeo wg = snd::make_wave_geo(s.nrows, s.ncols, s.dstate);
    const int pk = snd::wave_pack(wg, s.ncols);
    const int64_t waves = ((int64_t)s.batch * s.dim + pk - 1) / pk * wg.nseg;
    const bool shared = wg.nseg == 1 && waves >= 512;        // (wave_bwd_share() of the backward's launcher)
    const double t_row = pk == 8 ? (s.dstate <= 1 ? 0.75 : s.dstate == 2 ? 1.15 : 2.2) : pk > 1 ? (s.dstate <= 1 ? 0.65 : s.dstate == 2 ? 1.05 : 2.05)
                       : shared ? (s.dstate <= 1 ? 0.7 : s.dstate == 2 ? 1.15 : 2.4) : (s.dstate <= 1 ? 0.85 : s.dstate == 2 ? 1.5 : 2.95);
    // (a wide plane: one launch per column group of eight segments, one after the other)
    const double t_wave = (double)snd::wave_groups(wg.nsegAll) * (double)((waves + 2047) / 2048) * (wg.Hp + (wg.nseg - 1) * wg.R) * t_row;
    const int64_t blocks = plane_chunks(s);
    const double t_plane = (double)((blocks + 1023) / 1024) * g.nCX * g.nCY * 18.5;
    const int64_t rounds = (blocks * g.nCY + 1023) / 1024;
    const double steps = (double)rounds * g.nCX > g.nCX + g.nCY - 1 ? (double)rounds * g.nCX : g.nCX + g.nCY - 1;
    // (the tile kernels pipeline the strips of a plane only where use_strip_pipeline() says so)
    const bool pipelined = snd::use_strip_pipeline(snd::kSchedAuto, blocks, g.nCY, &s, g.nCX, snd::bwd_slots(s.dstate));
    return t_wave <= (pipelined ? steps * 25.0 : t_plane);
}

// Which kernel family a call runs: the row-segment wavefront when asked for, or under AUTO when the shape
// qualifies (1-4 states) and the model above prefers it; the tile kernels otherwise.
// -1: WAVEFRONT asked for a shape it does not cover.
int use_wavefront(const snd_shape &s, int schedule) {
    const bool fits = snd::wave_family_fits(s.ncols, s.dstate);
    if (schedule == SND_SCHED_WAVEFRONT) return fits ? 1 : -1;
    return schedule == SND_SCHED_AUTO && fits && wave_family_pays(s) ? 1 : 0;
}

// The kernels address inside one batch image with unsigned 32-bit BYTE offsets from a scalar base
// and form row offsets with 24-bit multiplies: a (count x stride) walk plus rows must stay below
// 2^32 bytes and a row pitch below 2^23 bytes.
int esize(int dt) { return dt == SND_F32 ? 4 : 2; }
bool fits32(int64_t a_count, int64_t a_stride, int64_t rows, int64_t h_stride, int64_t cols, int esz) {
    if (a_stride < 0 || h_stride < 0) return false;
    if (h_stride * esz >= ((int64_t)1 << 23) || rows >= ((int64_t)1 << 23) || cols >= ((int64_t)1 << 21)) return false;
    return ((a_count - 1) * a_stride + (rows - 1) * h_stride + cols) * esz < ((int64_t)1 << 32);
}

int check_fwd(const snd_fwd_params &p, bool need_state) {
    int st = check_shape(p.shape);
    if (st != SND_OK) return st;
    if (!p.u || !p.delta || !p.A || !p.B || !p.C) return SND_ERR_NULL;
    if (!p.x_v) return SND_ERR_WORKSPACE;
    if ((p.x == nullptr) != (p.x_sd == nullptr)) return SND_ERR_WORKSPACE;
    if (need_state && !p.x) return SND_ERR_WORKSPACE;
    if (!aligned16(p.x_v) || !aligned16(p.x) || !aligned16(p.x_sd)) return SND_ERR_ALIGN;
    if (p.u_h_stride < p.shape.ncols || p.delta_h_stride < p.shape.ncols || p.B_h_stride < p.shape.ncols ||
        p.C_h_stride < p.shape.ncols)
        if (p.shape.nrows > 1) return SND_ERR_STRIDE;
    const snd_shape &s = p.shape;
    const int e = esize(s.in_dtype);
    if ((p.u_shared != 0 && p.u_shared != 1) ||
        !fits32(p.u_shared ? s.dim / s.n_groups : s.dim, p.u_d_stride, s.nrows, p.u_h_stride, s.ncols, e) ||
        !fits32(s.delta_dim, p.delta_d_stride, s.nrows, p.delta_h_stride, s.ncols, e) ||
        !fits32(1, 0, s.nrows, p.B_h_stride, s.ncols, e) || p.B_dstate_stride < 0 ||
        !fits32(1, 0, s.nrows, p.C_h_stride, s.ncols, e) || p.C_dstate_stride < 0 ||
        !fits32(s.dim, (int64_t)s.nrows * s.ncols, s.nrows, s.ncols, s.ncols, 4))      // dense per-image gradients
        return SND_ERR_STRIDE;
    return SND_OK;
}

}  // namespace

extern "C" {

int snd_version(void) { return 210; }

const char *snd_status_string(int status) {
    switch (status) {
        case SND_OK: return "ok";
        case SND_ERR_NULL: return "a required pointer is null";
        case SND_ERR_SHAPE: return "bad shape: need dim % n_groups == 0, dim % delta_dim == 0, 1 <= dstate <= 16, all sizes > 0";
        case SND_ERR_DTYPE: return "unsupported dtype combination (inputs fp32/fp16/bf16; out and dout fp32 or the input dtype)";
        case SND_ERR_STRIDE: return "bad stride: rows must not overlap, the last dimension must be contiguous, one batch image must span fewer than 2^32 bytes and a row pitch fewer than 2^23 bytes";
        case SND_ERR_LAUNCH: return "kernel launch failed";
        case SND_ERR_WORKSPACE: return "saved state (x, x_v, x_sd) or workspace missing or too small";
        case SND_ERR_ALIGN: return "saved state / workspace pointers must be 16-byte aligned";
        case SND_ERR_TOO_LARGE: return "the problem needs more scratch than the static workspace holds (snd_static_workspace_bytes); use snd_bwd with a caller workspace";
        case SND_ERR_PIPELINE: return "a hand-over wait between blocks timed out in an earlier launch on this workspace: its outputs are NaN";
        default: return "unknown status";
    }
}

int snd_make_plan(const snd_shape *shape, snd_plan *plan) {
    if (!shape || !plan) return SND_ERR_NULL;
    int st = check_shape(*shape);
    if (st != SND_OK) return st;
    const snd::Geo g = snd::make_geo(shape->nrows, shape->ncols);
    const int64_t planes = (int64_t)shape->batch * shape->dim * shape->dstate;
    plan->n_chunks_x = g.nCX;
    plan->n_chunks_y = g.nCY;
    plan->x_inner = g.Hp;
    plan->xv_inner = g.Wp;
    const bool wave = snd::wave_family_fits(shape->ncols, shape->dstate);
    if (wave) {
        // either family may run on this shape: the inner extents grow until the wavefront layout fits too
        const snd::WaveGeo wg = snd::make_wave_geo(shape->nrows, shape->ncols, shape->dstate);
        const int64_t need_x = (snd::wave_x_plane(wg) + g.nCX - 1) / g.nCX, need_xv = (snd::wave_xv_plane(wg) + g.nCY - 1) / g.nCY;
        if (need_x > plan->x_inner) plan->x_inner = (int32_t)((need_x + 3) / 4 * 4);
        if (need_xv > plan->xv_inner) plan->xv_inner = (int32_t)((need_xv + 3) / 4 * 4);
    }
    plan->x_elems = planes * g.nCX * plan->x_inner;
    plan->x_sd_elems = plan->x_elems;
    plan->x_v_elems = planes * g.nCY * plan->xv_inner;
    // strip-pipeline sync words, then one row per plane: forward, h handed from a strip to the strip
    // below (strip schedule only); backward, the adjoint G = a*g handed to the strip above
    const int64_t sync_bytes = snd::sync_words(plane_chunks(*shape), g.nCY) * (int64_t)sizeof(int);
    const int64_t row_bytes = planes * (int64_t)g.Wp * (int64_t)sizeof(float);   // (tile layout: Wp = nCX * 8)
    plan->fwd_workspace_bytes = sync_bytes + row_bytes;      // the strip schedule's hand-over row of h
    plan->bwd_workspace_bytes = sync_bytes + row_bytes;      // the adjoint row G = a*g
    plan->wavefront_workspace = 0;
    plan->reserved_ = 0;
    if (wave && snd::wave_wide(shape->ncols, shape->dstate)) {
        plan->wavefront_workspace = 1;
        // wide planes under the row-segment kernels: what column groups hand over (behind the sync words, which stay
        // the tile kernels'): forward without saved state, a stand-in for x and x_sd; backward, G, Gs, a per boundary
        const snd::WaveGeo wg = snd::make_wave_geo(shape->nrows, shape->ncols, shape->dstate);
        const int64_t off = group_ws_offset(*shape);
        const int64_t fw = off + 2 * planes * snd::wave_x_plane(wg) * (int64_t)sizeof(float), bw = off + planes * snd::wave_bcol_plane(wg) * (int64_t)sizeof(float);
        if (fw > plan->fwd_workspace_bytes) plan->fwd_workspace_bytes = fw;
        if (bw > plan->bwd_workspace_bytes) plan->bwd_workspace_bytes = bw;
    }
    if (wave && snd::wave_bwd_split(shape->batch, shape->dim, shape->ncols, shape->dstate)) {
        // split planes (backward of the row-segment kernels): the tagged words the two halves of a plane hand over through
        plan->wavefront_workspace = 1;
        const snd::WaveGeo wg = snd::make_wave_geo(shape->nrows, shape->ncols, shape->dstate);
        const int64_t bw = group_ws_offset(*shape) + planes * snd::wave_split_words(wg) * (int64_t)sizeof(float);
        if (bw > plan->bwd_workspace_bytes) plan->bwd_workspace_bytes = bw;
    }
    // and, where the backward's strips are cut into column segments, one carried column state per strip
    if (snd::strip_segments(plane_chunks(*shape), g.nCY, g.nCX, snd::bwd_slots(shape->dstate), snd::job_queues(shape->batch * shape->n_groups)) > 1)
        plan->bwd_workspace_bytes += plane_chunks(*shape) * g.nCY * (int64_t)snd::kColStateFloats * (int64_t)sizeof(float);
    const int fwd_jobs = snd::fwd_band_count(SND_SCHED_AUTO, (int64_t)shape->batch * shape->n_groups,
                                             (shape->dim / shape->n_groups + 15) / 16, g.nCY, plan, shape->dstate, g.nCX);
    plan->auto_schedule = fwd_jobs == 0 ? SND_SCHED_PLANE : fwd_jobs == g.nCY ? SND_SCHED_STRIPS : SND_SCHED_BANDS;
    plan->auto_bwd_jobs = snd::bwd_band_count(SND_SCHED_AUTO, (int64_t)shape->batch * shape->n_groups,
                                              (shape->dim / shape->n_groups + 15) / 16, g.nCY, plan, shape->dstate, g.nCX);
    if (wave && wave_family_pays(*shape)) {
        plan->auto_schedule = SND_SCHED_WAVEFRONT;
        plan->auto_bwd_jobs = 0;
    }
    // Placement advice (see the header).  Measured on dC - dB modulo the fp32 row of dB/dC: the row-segment
    // backward is fastest half a row apart when a row is 2 KiB or more (512 x 512: 0.46 ms at 1 KiB + k * 2 KiB,
    // 0.55 at k * 2 KiB), and with narrower rows at 16 KiB (0 .. 9 KiB cost some shapes 10 % and gain others as much);
    // the tile kernels are indifferent.
    // With three or four states and rows of 2 KiB or more no distance beat none at all (2 x 64 x 256x512, four states:
    // 0.69 ms at 0, 0.77 half a row apart; 256x1024: 1.81 against 2.17).
    const int64_t row = (int64_t)shape->ncols * 4;
    plan->dC_skew_bytes = plan->auto_schedule != SND_SCHED_WAVEFRONT ? 5 * 1024
                        : row < 2048 ? 16 * 1024 : shape->dstate >= 3 ? 0 : (row / 2 + 255) / 256 * 256;
    return SND_OK;
}

int snd_fwd(const snd_fwd_params *params, snd_stream_t stream) {
    if (!params) return SND_ERR_NULL;
    int st = check_fwd(*params, false);
    if (st != SND_OK) return st;
    if (!params->out) return SND_ERR_NULL;
    if (params->out_dtype != SND_F32 && params->out_dtype != params->shape.in_dtype) return SND_ERR_DTYPE;
    if (params->merge != 0 && params->merge != 1) return SND_ERR_SHAPE;
    if (params->merge && params->out_dtype != SND_F32) return SND_ERR_DTYPE;   // accumulated with float atomics
    if (!fits32(params->merge ? params->shape.dim / params->shape.n_groups : params->shape.dim, params->out_d_stride,
                params->shape.nrows, params->out_h_stride, params->shape.ncols, esize(params->out_dtype)))
        return SND_ERR_STRIDE;
    if (params->schedule < SND_SCHED_AUTO || params->schedule > SND_SCHED_WAVEFRONT) return SND_ERR_SHAPE;
    if (params->directions != SND_DIR_TOPLEFT && params->directions != SND_DIR_CORNERS) return SND_ERR_SHAPE;
    int wave = use_wavefront(params->shape, params->schedule);
    if (wave < 0) return SND_ERR_SHAPE;
    float *group_ws = nullptr;
    if (wave && snd::wave_wide(params->shape.ncols, params->shape.dstate)) {
        // a wide plane's column groups hand over through the saved state, or without one through the workspace
        snd_plan plan;
        snd_make_plan(&params->shape, &plan);
        if (params->workspace && params->workspace_bytes >= plan.fwd_workspace_bytes) {
            if (!aligned16(params->workspace)) return SND_ERR_ALIGN;
            group_ws = (float *)((char *)params->workspace + group_ws_offset(params->shape));
        } else if (!params->x) {
            if (params->schedule == SND_SCHED_WAVEFRONT) return SND_ERR_WORKSPACE;
            wave = 0;                               // (AUTO: the tile kernels need neither)
        }
    }
    if (wave) {                                     // (other planes need no workspace)
        switch (params->shape.in_dtype) {
            case SND_F32: return snd::launch_wave_fwd_f32(*params, group_ws, (hipStream_t)stream);
            case SND_BF16: return snd::launch_wave_fwd_bf16(*params, group_ws, (hipStream_t)stream);
            default: return snd::launch_wave_fwd_f16(*params, group_ws, (hipStream_t)stream);
        }
    }
    if (params->workspace) {
        snd_plan plan;
        snd_make_plan(&params->shape, &plan);
        if (params->workspace_bytes < plan.fwd_workspace_bytes) return SND_ERR_WORKSPACE;
        if (!aligned16(params->workspace)) return SND_ERR_ALIGN;
    } else if (params->schedule == SND_SCHED_STRIPS || params->schedule == SND_SCHED_BANDS) {
        return SND_ERR_WORKSPACE;
    }
    switch (params->shape.in_dtype) {
        case SND_F32: return snd::launch_fwd_f32(*params, (hipStream_t)stream);
        case SND_BF16: return snd::launch_fwd_bf16(*params, (hipStream_t)stream);
        default: return snd::launch_fwd_f16(*params, (hipStream_t)stream);
    }
}

static int bwd_checked(const snd_bwd_params *params, snd_stream_t stream) {
    if (!params) return SND_ERR_NULL;
    int st = check_fwd(params->f, true);
    if (st != SND_OK) return st;
    if (!params->dout || !params->du || !params->ddelta || !params->dA || !params->dB || !params->dC)
        return SND_ERR_NULL;
    if (params->dout_dtype != SND_F32 && params->dout_dtype != params->f.shape.in_dtype) return SND_ERR_DTYPE;
    if ((params->f.D != nullptr) != (params->dD != nullptr)) return SND_ERR_NULL;
    if ((params->f.delta_bias != nullptr) != (params->ddelta_bias != nullptr)) return SND_ERR_NULL;
    if ((params->f.A_decay != nullptr) != (params->dA_decay != nullptr)) return SND_ERR_NULL;
    snd_plan plan;
    st = snd_make_plan(&params->f.shape, &plan);
    if (st != SND_OK) return st;
    if (params->f.schedule < SND_SCHED_AUTO || params->f.schedule > SND_SCHED_WAVEFRONT) return SND_ERR_SHAPE;
    if (params->f.directions != SND_DIR_TOPLEFT && params->f.directions != SND_DIR_CORNERS) return SND_ERR_SHAPE;
    if (params->f.merge != 0 && params->f.merge != 1) return SND_ERR_SHAPE;
    if (!fits32(params->f.merge ? params->f.shape.dim / params->f.shape.n_groups : params->f.shape.dim, params->dout_d_stride,
                params->f.shape.nrows, params->dout_h_stride, params->f.shape.ncols, esize(params->dout_dtype)))
        return SND_ERR_STRIDE;
    const int wave = use_wavefront(params->f.shape, params->f.schedule);
    if (wave < 0) return SND_ERR_SHAPE;
    float *group_ws = nullptr;
    if (wave && snd::wave_wide(params->f.shape.ncols, params->f.shape.dstate)) {   // a wide plane's column groups hand over here
        if (!params->workspace || params->workspace_bytes < plan.bwd_workspace_bytes) return SND_ERR_WORKSPACE;
        if (!aligned16(params->workspace)) return SND_ERR_ALIGN;
        group_ws = (float *)((char *)params->workspace + group_ws_offset(params->f.shape));
    } else if (wave && snd::wave_bwd_split(params->f.shape.batch, params->f.shape.dim, params->f.shape.ncols, params->f.shape.dstate) &&
               params->workspace && params->workspace_bytes >= plan.bwd_workspace_bytes && aligned16(params->workspace)) {
        // split planes: the faster backward where the caller brought the workspace for it, whole planes otherwise
        group_ws = (float *)((char *)params->workspace + group_ws_offset(params->f.shape));
    }
    if (wave) {                                     // (other planes need no workspace)
        // the row-segment backward addresses a batch image of du / ddelta and a (batch, group)'s dB / dC planes through
        // buffer descriptors: unsigned 32-bit byte offsets that must stay below the out-of-range marker
        const snd_shape &ws = params->f.shape;
        if ((int64_t)ws.dim * ws.nrows * ws.ncols * 4 >= (int64_t)snd::kBufOOB || (int64_t)ws.dstate * ws.nrows * ws.ncols * 4 >= (int64_t)snd::kBufOOB)
            return SND_ERR_STRIDE;
        switch (params->f.shape.in_dtype) {
            case SND_F32: return snd::launch_wave_bwd_f32(*params, group_ws, (hipStream_t)stream);
            case SND_BF16: return snd::launch_wave_bwd_bf16(*params, group_ws, (hipStream_t)stream);
            default: return snd::launch_wave_bwd_f16(*params, group_ws, (hipStream_t)stream);
        }
    }
    if (!params->workspace || params->workspace_bytes < plan.bwd_workspace_bytes) return SND_ERR_WORKSPACE;
    if (!aligned16(params->workspace)) return SND_ERR_ALIGN;
    switch (params->f.shape.in_dtype) {
        case SND_F32: return snd::launch_bwd_f32(*params, (hipStream_t)stream);
        case SND_BF16: return snd::launch_bwd_bf16(*params, (hipStream_t)stream);
        default: return snd::launch_bwd_f16(*params, (hipStream_t)stream);
    }
}

int snd_bwd(const snd_bwd_params *params, snd_stream_t stream) { return bwd_checked(params, stream); }

int snd_init(int device) {
    int cur = 0;
    if (hipGetDevice(&cur) != hipSuccess) return SND_ERR_LAUNCH;
    if (device != cur && hipSetDevice(device) != hipSuccess) return SND_ERR_LAUNCH;
    const int st = snd::ensure_device_ready();
    if (device != cur && hipSetDevice(cur) != hipSuccess) return SND_ERR_LAUNCH;
    return st;
}

int64_t snd_static_workspace_bytes(void) { return SND_STATIC_WORKSPACE_BYTES; }

int snd_bwd_static(const snd_bwd_params *params, snd_stream_t stream) {
    if (!params) return SND_ERR_NULL;
    snd_plan plan;
    int st = snd_make_plan(&params->f.shape, &plan);
    if (st != SND_OK) return st;
    // (the row-segment kernels use no scratch at all, wide planes aside: no size limit for them)
    const int wave = use_wavefront(params->f.shape, params->f.schedule);
    const bool scratch = wave == 0 || snd::wave_wide(params->f.shape.ncols, params->f.shape.dstate);
    if (scratch && plan.bwd_workspace_bytes > SND_STATIC_WORKSPACE_BYTES) return SND_ERR_TOO_LARGE;
    st = snd::ensure_device_ready();                // no allocation: symbol lookup and kernel attributes, once per device
    if (st != SND_OK) return st;
    void *ws = snd::device_scratch();
    if (!ws) return SND_ERR_LAUNCH;
    snd_bwd_params q = *params;
    q.workspace = ws;
    q.workspace_bytes = SND_STATIC_WORKSPACE_BYTES;
    return bwd_checked(&q, stream);
}

int snd_workspace_error(const void *workspace, snd_stream_t stream) {
    if (!workspace) {                               // the static scratch of snd_bwd_static on the current device
        workspace = snd::device_scratch();
        if (!workspace) return SND_ERR_NULL;        // (never set up: no launch has used it)
    }
    int word = 0;
    if (hipMemcpyAsync(&word, (const int *)workspace + snd::kErrorWord, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess)
        return SND_ERR_LAUNCH;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return SND_ERR_LAUNCH;
    return word != 0 ? SND_ERR_PIPELINE : SND_OK;
}

void snd_debug_set_strip_slots(int slots) { snd::g_strip_slots.store(slots, std::memory_order_relaxed); }

void snd_debug_set_spin_limit(int polls) { snd::g_spin_limit.store(polls > 0 ? polls : snd::kSpinLimit, std::memory_order_relaxed); }

}  // extern "C"
