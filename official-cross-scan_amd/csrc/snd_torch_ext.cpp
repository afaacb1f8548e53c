// Thin PyTorch-ROCm extension over the C ABI in include/snd_scan.h.
//
// Exports the reference's operator pair with the reference's argument and return lists
// (kernels/selective_nd_scan/src/cusoflex/selective_scan_oflex.cpp:179-187,282 and :286-297,432-438,
// pybind :442-445):
//     fwd(u, delta, A, B, C, D?, delta_bias?, delta_softplus, out_float, A_decay?) -> [out, x, x_v, x_sd]
//     bwd(u, delta, A, B, C, D?, delta_bias?, dout, x?, x_v?, delta_softplus, A_decay?, x_sd?)
//         -> [du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay]
// It does what a host binding has to do and nothing else: the reference's TORCH_CHECKs
// (:188-245, :298-391), allocation of outputs / saved state / scratch, device guard, current-stream
// lookup, and mapping of a non-zero library status to a c10::Error (Python RuntimeError).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <atomic>
#include <cstdlib>
#include <vector>

#include "snd_scan.h"

namespace {

#define CHECK_SHAPE(x, ...) \
    TORCH_CHECK(x.sizes() == torch::IntArrayRef({__VA_ARGS__}), #x " must have shape (" #__VA_ARGS__ ")")

// bytes rounded up to the 2 MiB grid that large allocations start on (the grid snd_plan's placement advice refers to)
int64_t round_2mib(int64_t bytes) { return (bytes + (2 << 20) - 1) / (2 << 20) * (2 << 20); }

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::ScalarType::Float: return SND_F32;
        case at::ScalarType::Half: return SND_F16;
        case at::ScalarType::BFloat16: return SND_BF16;
        default: TORCH_CHECK(false, "selective_nd_scan: unsupported dtype ", toString(t)); return -1;
    }
}

void check_status(int st, const char *what) {
    TORCH_CHECK(st == SND_OK, "selective_nd_scan ", what, " failed: ", snd_status_string(st), " (status ", st, ")");
}

struct Checked {
    int batch, dim, nrows, ncols, dstate, n_groups, delta_dim;
    bool u_shared;                 // u is [batch, dim / n_groups, H, W]: one feature map scanned by every group
    snd_shape shape;
    snd_plan plan;
};

// The checks of selective_scan_oflex.cpp:188-245 (shared by fwd and bwd).
Checked check_inputs(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A, const at::Tensor &B,
                     const at::Tensor &C, const c10::optional<at::Tensor> &D_,
                     const c10::optional<at::Tensor> &delta_bias_, const c10::optional<at::Tensor> &A_decay_) {
    auto input_type = u.scalar_type();
    TORCH_CHECK(input_type == at::ScalarType::Float || input_type == at::ScalarType::Half ||
                input_type == at::ScalarType::BFloat16, "u must be float32, float16 or bfloat16");
    TORCH_CHECK(A.scalar_type() == at::ScalarType::Float, "A must be float32");
    TORCH_CHECK(delta.scalar_type() == input_type && B.scalar_type() == input_type && C.scalar_type() == input_type,
                "u, delta, B, C must share one dtype");
    TORCH_CHECK(u.is_cuda() && delta.is_cuda() && A.is_cuda() && B.is_cuda() && C.is_cuda(),
                "all tensors must be on the GPU");
    TORCH_CHECK(u.dim() == 4 && delta.dim() == 4 && A.dim() == 2 && B.dim() == 5 && C.dim() == 5,
                "expected u, delta 4-D; A 2-D; B, C 5-D");
    TORCH_CHECK(u.stride(-1) == 1 || u.size(-1) == 1, "u must be contiguous in its last dimension");
    TORCH_CHECK(delta.stride(-1) == 1 || delta.size(-1) == 1, "delta must be contiguous in its last dimension");

    Checked c;
    // dim is A's (the reference takes it from u, selective_scan_oflex.cpp:206): u may carry only
    // dim / n_groups channels, shared by all groups (the CrossScan of one feature map without copies)
    c.batch = u.size(0); c.dim = A.size(0); c.nrows = u.size(2); c.ncols = u.size(3);
    c.dstate = A.size(1); c.n_groups = B.size(1); c.delta_dim = delta.size(1);
    c.u_shared = u.size(1) != c.dim;
    TORCH_CHECK(!c.u_shared || u.size(1) * c.n_groups == c.dim,
                "u must have dim = A.size(0) channels, or dim / n_groups channels shared by the groups");
    TORCH_CHECK(c.dim % c.n_groups == 0, "dims should be dividable by n_groups");
    TORCH_CHECK(c.dim % c.delta_dim == 0, "dims should be dividable by delta_dim");
    TORCH_CHECK(c.dstate <= SND_MAX_DSTATE, "selective_scan only supports state dimension <= 16");
    const int batch_size = c.batch, dim = c.dim, nrows = c.nrows, ncols = c.ncols, dstate = c.dstate,
              n_groups = c.n_groups, delta_dim = c.delta_dim;
    CHECK_SHAPE(u, batch_size, c.u_shared ? dim / n_groups : dim, nrows, ncols);
    CHECK_SHAPE(delta, batch_size, delta_dim, nrows, ncols);
    CHECK_SHAPE(A, dim, dstate);
    CHECK_SHAPE(B, batch_size, n_groups, dstate, nrows, ncols);
    TORCH_CHECK(B.stride(-1) == 1 || B.size(-1) == 1, "B must be contiguous in its last dimension");
    CHECK_SHAPE(C, batch_size, n_groups, dstate, nrows, ncols);
    TORCH_CHECK(C.stride(-1) == 1 || C.size(-1) == 1, "C must be contiguous in its last dimension");
    if (A_decay_.has_value()) {
        const auto &A_decay = A_decay_.value();
        TORCH_CHECK(A_decay.scalar_type() == at::ScalarType::Float && A_decay.is_cuda());
        CHECK_SHAPE(A_decay, 1);
    }
    if (D_.has_value()) {
        const auto &D = D_.value();
        TORCH_CHECK(D.scalar_type() == at::ScalarType::Float && D.is_cuda());
        TORCH_CHECK(D.stride(-1) == 1 || D.size(-1) == 1);
        CHECK_SHAPE(D, dim);
    }
    if (delta_bias_.has_value()) {
        const auto &delta_bias = delta_bias_.value();
        TORCH_CHECK(delta_bias.scalar_type() == at::ScalarType::Float && delta_bias.is_cuda());
        TORCH_CHECK(delta_bias.stride(-1) == 1 || delta_bias.size(-1) == 1);
        CHECK_SHAPE(delta_bias, delta_dim);
    }
    c.shape = snd_shape{c.batch, c.dim, c.nrows, c.ncols, c.dstate, c.n_groups, c.delta_dim, dtype_code(input_type)};
    check_status(snd_make_plan(&c.shape, &c.plan), "plan");
    return c;
}

// Default snd_schedule of fwd and bwd (0 = chosen by shape) when a call does not name one; set_schedule()
// is for tests and tuning.  Calls that pass `schedule` themselves never read it.
std::atomic<int> g_schedule{SND_SCHED_AUTO};
// Opt-in check of the pipelined schedules' error word after every launch (costs a stream sync):
// SND_CHECK_PIPELINE=1 in the environment, or set_debug(True).
std::atomic<bool> g_check_pipeline{[] { const char *e = std::getenv("SND_CHECK_PIPELINE"); return e && e[0] && e[0] != '0'; }()};

int resolve_schedule(int64_t schedule) {
    if (schedule < 0) return g_schedule.load();
    TORCH_CHECK(schedule >= SND_SCHED_AUTO && schedule <= SND_SCHED_WAVEFRONT,
                "schedule must be 0 (auto), 1 (plane), 2 (strips), 3 (bands) or 4 (row-segment wavefront)");
    return (int)schedule;
}
// whether a call with this schedule runs one of the pipelined tile schedules (they need the workspace)
bool pipelined(int sched, int auto_choice) {
    const int s = sched == SND_SCHED_AUTO ? auto_choice : sched;
    return s == SND_SCHED_STRIPS || s == SND_SCHED_BANDS;
}
bool wavefront(int sched, const snd_plan &plan) {
    return sched == SND_SCHED_WAVEFRONT || (sched == SND_SCHED_AUTO && plan.auto_schedule == SND_SCHED_WAVEFRONT);
}
void check_pipeline(const at::Tensor &ws, hipStream_t stream, const char *what) {
    if (!ws.defined() || !g_check_pipeline.load()) return;
    const int st = snd_workspace_error(ws.data_ptr(), (snd_stream_t)stream);
    TORCH_CHECK(st == SND_OK, "selective_nd_scan ", what, ": ", snd_status_string(st), " (status ", st, ")");
}

void fill_fwd(snd_fwd_params &p, const Checked &c, const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
              const at::Tensor &B, const at::Tensor &C, const c10::optional<at::Tensor> &D_,
              const c10::optional<at::Tensor> &delta_bias_, const c10::optional<at::Tensor> &A_decay_,
              bool delta_softplus) {
    memset(&p, 0, sizeof(p));
    p.shape = c.shape;
    p.u_shared = c.u_shared ? 1 : 0;
    p.delta_softplus = delta_softplus ? 1 : 0;
    p.u = u.data_ptr(); p.delta = delta.data_ptr(); p.B = B.data_ptr(); p.C = C.data_ptr();
    p.A = A.data_ptr<float>();
    p.D = D_.has_value() ? D_.value().data_ptr<float>() : nullptr;
    p.delta_bias = delta_bias_.has_value() ? delta_bias_.value().data_ptr<float>() : nullptr;
    p.A_decay = A_decay_.has_value() ? A_decay_.value().data_ptr<float>() : nullptr;
    p.u_batch_stride = u.stride(0); p.u_d_stride = u.stride(1); p.u_h_stride = u.stride(2);
    p.delta_batch_stride = delta.stride(0); p.delta_d_stride = delta.stride(1); p.delta_h_stride = delta.stride(2);
    p.A_d_stride = A.stride(0); p.A_dstate_stride = A.stride(1);
    p.B_batch_stride = B.stride(0); p.B_group_stride = B.stride(1); p.B_dstate_stride = B.stride(2); p.B_h_stride = B.stride(3);
    p.C_batch_stride = C.stride(0); p.C_group_stride = C.stride(1); p.C_dstate_stride = C.stride(2); p.C_h_stride = C.stride(3);
}

// Fused CrossMerge arguments: weights are one float32 per channel, contiguous, on the inputs' device.
void check_merge(const Checked &c, bool merge, const c10::optional<at::Tensor> &w, const at::Tensor &u) {
    if (!merge) {
        TORCH_CHECK(!w.has_value(), "merge_weights given without merge=True");
        return;
    }
    if (w.has_value()) {
        const at::Tensor &t = w.value();
        TORCH_CHECK(t.scalar_type() == at::ScalarType::Float && t.is_cuda() && t.is_contiguous() && t.numel() == c.dim &&
                        t.device() == u.device(),
                    "merge_weights must be a contiguous float32 GPU tensor with dim = ", c.dim, " elements");
    }
}

std::vector<at::Tensor> selective_scan_fwd(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
                                           const at::Tensor &B, const at::Tensor &C,
                                           const c10::optional<at::Tensor> &D_,
                                           const c10::optional<at::Tensor> &delta_bias_, bool delta_softplus,
                                           bool out_float, const c10::optional<at::Tensor> &A_decay_,
                                           int64_t directions, int64_t schedule, bool merge,
                                           const c10::optional<at::Tensor> &merge_weights_) {
    TORCH_CHECK(directions == SND_DIR_TOPLEFT || directions == SND_DIR_CORNERS, "directions must be 0 (top-left) or 1 (four corners)");
    const Checked c = check_inputs(u, delta, A, B, C, D_, delta_bias_, A_decay_);
    check_merge(c, merge, merge_weights_, u);
    TORCH_CHECK(!merge || out_float, "the fused merge accumulates in float32: out_float must be true");
    at::hip::HIPGuardMasqueradingAsCUDA device_guard{u.device()};
    const auto f32 = u.options().dtype(at::ScalarType::Float);
    // merged: one fp32 channel per feature, zero-filled, to which every group adds its weighted result
    at::Tensor out = merge ? torch::zeros({c.batch, c.dim / c.n_groups, c.nrows, c.ncols}, f32)
                           : torch::empty({c.batch, c.dim, c.nrows, c.ncols},
                                          u.options().dtype(out_float ? at::ScalarType::Float : u.scalar_type()));
    at::Tensor x = torch::empty({c.batch, c.dim, c.dstate, c.plan.n_chunks_x, c.plan.x_inner}, f32);
    at::Tensor x_v = torch::empty({c.batch, c.dim, c.dstate, c.plan.n_chunks_y, c.plan.xv_inner}, f32);
    at::Tensor x_sd = torch::empty({c.batch, c.dim, c.dstate, c.plan.n_chunks_x, c.plan.x_inner}, f32);

    snd_fwd_params p;
    fill_fwd(p, c, u, delta, A, B, C, D_, delta_bias_, A_decay_, delta_softplus);
    p.out = out.data_ptr();
    p.out_dtype = dtype_code(out.scalar_type());
    p.out_batch_stride = out.stride(0); p.out_d_stride = out.stride(1); p.out_h_stride = out.stride(2);
    p.x = x.data_ptr<float>(); p.x_v = x_v.data_ptr<float>(); p.x_sd = x_sd.data_ptr<float>();
    // scratch for the strip-pipelined schedule (only when it will be used); released to the caching
    // allocator in stream order
    const int sched = resolve_schedule(schedule);
    p.schedule = sched;
    at::Tensor ws;
    if (pipelined(sched, c.plan.auto_schedule)) {
        ws = torch::empty({(c.plan.fwd_workspace_bytes + 3) / 4}, f32);
        p.workspace = ws.data_ptr();
        p.workspace_bytes = c.plan.fwd_workspace_bytes;
    }
    p.directions = (int32_t)directions;
    p.merge = merge ? 1 : 0;
    p.merge_weights = merge && merge_weights_.has_value() ? merge_weights_.value().data_ptr<float>() : nullptr;
    auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_status(snd_fwd(&p, (snd_stream_t)stream), "fwd");
    check_pipeline(ws, stream, "fwd");
    return {out, x, x_v, x_sd};
}

std::vector<at::Tensor> selective_scan_bwd(const at::Tensor &u, const at::Tensor &delta, const at::Tensor &A,
                                           const at::Tensor &B, const at::Tensor &C,
                                           const c10::optional<at::Tensor> &D_,
                                           const c10::optional<at::Tensor> &delta_bias_, const at::Tensor &dout,
                                           const c10::optional<at::Tensor> &x_, const c10::optional<at::Tensor> &x_v_,
                                           bool delta_softplus, const c10::optional<at::Tensor> &A_decay_,
                                           const c10::optional<at::Tensor> &x_sd_, int64_t directions, int64_t schedule,
                                           bool merge, const c10::optional<at::Tensor> &merge_weights_) {
    TORCH_CHECK(directions == SND_DIR_TOPLEFT || directions == SND_DIR_CORNERS, "directions must be 0 (top-left) or 1 (four corners)");
    const Checked c = check_inputs(u, delta, A, B, C, D_, delta_bias_, A_decay_);
    check_merge(c, merge, merge_weights_, u);
    const int batch_size = c.batch, dim = c.dim, nrows = c.nrows, ncols = c.ncols, dstate = c.dstate;
    TORCH_CHECK(dout.scalar_type() == u.scalar_type() || dout.scalar_type() == at::ScalarType::Float,
                "dout must be float32 or the input dtype");
    TORCH_CHECK(dout.is_cuda());
    TORCH_CHECK(dout.stride(-1) == 1 || dout.size(-1) == 1, "dout must be contiguous in its last dimension");
    CHECK_SHAPE(dout, batch_size, merge ? dim / c.n_groups : dim, nrows, ncols);   // merged: the gradient of the merged output
    // the saved state is required: gradients computed without it would belong to another function
    TORCH_CHECK(x_.has_value() && x_v_.has_value() && x_sd_.has_value(),
                "bwd needs the x, x_v and x_sd tensors returned by fwd");
    const auto &x = x_.value(), &x_v = x_v_.value(), &x_sd = x_sd_.value();
    const int nChunksX = c.plan.n_chunks_x, nChunksY = c.plan.n_chunks_y, x_inner = c.plan.x_inner,
              xv_inner = c.plan.xv_inner;
    for (const at::Tensor *t : {&x, &x_v, &x_sd}) {
        TORCH_CHECK(t->scalar_type() == at::ScalarType::Float && t->is_cuda() && t->is_contiguous(),
                    "saved state must be contiguous float32 GPU tensors");
    }
    CHECK_SHAPE(x, batch_size, dim, dstate, nChunksX, x_inner);
    CHECK_SHAPE(x_sd, batch_size, dim, dstate, nChunksX, x_inner);
    CHECK_SHAPE(x_v, batch_size, dim, dstate, nChunksY, xv_inner);

    at::hip::HIPGuardMasqueradingAsCUDA device_guard{u.device()};
    const auto f32 = u.options().dtype(at::ScalarType::Float);
    at::Tensor du = torch::empty({batch_size, dim, nrows, ncols}, u.options());
    at::Tensor ddelta = torch::empty({batch_size, dim, nrows, ncols}, u.options());
    // the accumulated gradients are zero-filled as host.cpp:395-403 does.  dB and dC share one buffer (one
    // fill kernel for the two large tensors); the small ones (dA, dD, ddelta_bias, dA_decay) share another,
    // so that a parameter gradient kept by the optimizer never pins the large buffer.
    const int64_t nA = (int64_t)dim * dstate, nBC = B.numel();
    auto round64 = [](int64_t v) { return (v + 63) / 64 * 64; };
    // dB and dC are accumulated at equal offsets at the same time.  Where that matters (the row-segment kernels on
    // tensors of 2 MiB and more) dC starts a chosen distance past the 2 MiB-rounded end of dB (snd_plan.dC_skew_bytes:
    // not a multiple of 2 MiB apart); everywhere else it follows dB directly and nothing beyond the two is filled.
    const bool spread = c.plan.auto_schedule == SND_SCHED_WAVEFRONT && nBC * 4 >= (int64_t)(2 << 20);
    const int64_t oC = spread ? (round_2mib(nBC * 4) + c.plan.dC_skew_bytes) / 4 : round64(nBC);
    // one fill (and, for 16-bit inputs, one cast) over both where the gap between them is small beside them, else one
    // per tensor
    const bool whole = (oC - nBC) * 4 <= nBC;
    at::Tensor accBC = whole ? torch::zeros({oC + nBC}, f32) : torch::empty({oC + nBC}, f32);
    at::Tensor dB = accBC.narrow(0, 0, nBC).view(B.sizes());
    at::Tensor dC = accBC.narrow(0, oC, nBC).view(C.sizes());
    if (!whole) { dB.zero_(); dC.zero_(); }         // (not the gap between them)
    const int64_t oD = round64(nA), oBias = oD + round64(dim), oDec = oBias + round64(dim), oMerge = oDec + 64;
    at::Tensor accP = torch::zeros({oMerge + (merge ? round64(dim) : 0)}, f32);
    at::Tensor dA = accP.narrow(0, 0, nA).view({dim, dstate});
    at::Tensor dD, ddelta_bias, dA_decay;
    if (D_.has_value()) dD = accP.narrow(0, oD, dim);
    if (delta_bias_.has_value()) ddelta_bias = accP.narrow(0, oBias, dim);
    if (A_decay_.has_value()) dA_decay = accP.narrow(0, oDec, 1);
    at::Tensor dmerge;                              // weight * d(weight) per channel (the caller divides)
    if (merge) dmerge = accP.narrow(0, oMerge, dim);
    const int sched = resolve_schedule(schedule);
    at::Tensor ws;                                  // the wavefront kernels need none, except for planes taken in column groups
    if (!wavefront(sched, c.plan) || c.plan.wavefront_workspace) ws = torch::empty({(c.plan.bwd_workspace_bytes + 3) / 4}, f32);

    snd_bwd_params p;
    memset(&p, 0, sizeof(p));
    fill_fwd(p.f, c, u, delta, A, B, C, D_, delta_bias_, A_decay_, delta_softplus);
    p.f.x = x.data_ptr<float>(); p.f.x_v = x_v.data_ptr<float>(); p.f.x_sd = x_sd.data_ptr<float>();
    p.dout = dout.data_ptr();
    p.dout_dtype = dtype_code(dout.scalar_type());
    p.dout_batch_stride = dout.stride(0); p.dout_d_stride = dout.stride(1); p.dout_h_stride = dout.stride(2);
    p.du = du.data_ptr(); p.ddelta = ddelta.data_ptr();
    p.dA = dA.data_ptr<float>(); p.dB = dB.data_ptr<float>(); p.dC = dC.data_ptr<float>();
    p.dD = dD.defined() ? dD.data_ptr<float>() : nullptr;
    p.ddelta_bias = ddelta_bias.defined() ? ddelta_bias.data_ptr<float>() : nullptr;
    p.dA_decay = dA_decay.defined() ? dA_decay.data_ptr<float>() : nullptr;
    p.workspace = ws.defined() ? ws.data_ptr() : nullptr;
    p.workspace_bytes = ws.defined() ? c.plan.bwd_workspace_bytes : 0;
    p.f.schedule = sched;
    p.f.directions = (int32_t)directions;
    p.f.merge = merge ? 1 : 0;
    p.f.merge_weights = merge && merge_weights_.has_value() ? merge_weights_.value().data_ptr<float>() : nullptr;
    p.dmerge = dmerge.defined() ? dmerge.data_ptr<float>() : nullptr;
    auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    check_status(snd_bwd(&p, (snd_stream_t)stream), "bwd");
    if (sched == SND_SCHED_STRIPS || sched == SND_SCHED_BANDS || (sched == SND_SCHED_AUTO && c.plan.auto_bwd_jobs != 0))
        check_pipeline(ws, stream, "bwd");

    // host.cpp:432-438: cast dB/dC to the input dtype, fold channel groups that share a delta
    // (16-bit inputs: one cast kernel for the two tensors, which share a buffer)
    at::Tensor dBo = dB, dCo = dC;
    if (B.scalar_type() != at::ScalarType::Float) {
        if (!whole) {                               // two casts of the live ranges, not one of the gap as well
            dBo = dB.to(B.dtype());
            dCo = dC.to(C.dtype());
        } else {
            const at::Tensor cast = accBC.to(B.dtype());
            dBo = cast.narrow(0, 0, nBC).view(B.sizes());
            dCo = cast.narrow(0, oC, nBC).view(C.sizes());
        }
    }
    std::vector<at::Tensor> result = {du, ddelta, dA, dBo, dCo, dD, ddelta_bias, dA_decay};
    if (dim != c.delta_dim) {
        const int rep = dim / c.delta_dim;
        result[1] = ddelta.view({batch_size, c.delta_dim, rep, nrows, ncols}).sum(2);
        if (delta_bias_.has_value()) result[6] = ddelta_bias.view({c.delta_dim, rep}).sum(1);
    }
    if (c.u_shared)   // one feature map scanned by every group: its gradient is the sum over the groups
        result[0] = du.view({batch_size, c.n_groups, dim / c.n_groups, nrows, ncols}).sum(1);
    if (merge) result.push_back(dmerge);
    return result;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    // the reference's positional lists (selective_scan_oflex.cpp:179-187,286-297) plus trailing optional
    // arguments: the per-group scan origin the reference leaves as a TODO (fwd.cuh:140), the block mapping
    // of this call (-1: the module default), and the fused CrossMerge (out / dout have dim / n_groups
    // channels, merge_weights [dim] float32 or None for the plain sum; bwd then returns a ninth tensor,
    // merge_weights * d merge_weights per channel)
    namespace py = pybind11;
    m.def("fwd", &selective_scan_fwd, "Selective nd scan forward (gfx950)", py::arg("u"), py::arg("delta"), py::arg("A"),
          py::arg("B"), py::arg("C"), py::arg("D"), py::arg("delta_bias"), py::arg("delta_softplus"), py::arg("out_float"),
          py::arg("A_decay"), py::arg("directions") = 0, py::arg("schedule") = -1, py::arg("merge") = false,
          py::arg("merge_weights") = py::none());
    m.def("bwd", &selective_scan_bwd, "Selective nd scan backward (gfx950)", py::arg("u"), py::arg("delta"), py::arg("A"),
          py::arg("B"), py::arg("C"), py::arg("D"), py::arg("delta_bias"), py::arg("dout"), py::arg("x"), py::arg("x_v"),
          py::arg("delta_softplus"), py::arg("A_decay"), py::arg("x_sd"), py::arg("directions") = 0, py::arg("schedule") = -1,
          py::arg("merge") = false, py::arg("merge_weights") = py::none());
    m.def("set_schedule", [](int mode) {
        TORCH_CHECK(mode >= SND_SCHED_AUTO && mode <= SND_SCHED_WAVEFRONT, "schedule must be 0 (auto), 1 (plane), 2 (strips), 3 (bands) or 4 (row-segment wavefront)");
        g_schedule.store(mode);
    }, "Default block mapping of calls that pass no schedule: 0 auto, 1 one block per plane chunk, 2 pipelined row strips, 3 bands");
    m.def("get_schedule", [] { return g_schedule.load(); }, "The default block mapping calls use when they name none (see set_schedule)");
    m.def("set_debug", [](bool on) { g_check_pipeline.store(on); },
          "Check the pipelined schedules' error word after every launch (a stream sync per call) and raise if a hand-over wait timed out");
    m.def("init", [](int device) { check_status(snd_init(device), "init"); },
          "Per-device set-up (kernel attributes); call once before capturing launches into a HIP graph");
}
