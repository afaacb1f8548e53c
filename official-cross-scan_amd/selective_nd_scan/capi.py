"""ctypes binding of include/snd_scan.h: the C ABI driven as a foreign host would drive it, with
plain pointers, sizes and a stream (torch only owns the device memory).

Used by the parity tests and by the benchmark's kernel-only timing; the operator that models call
goes through the C++ extension instead (interface.py).
"""
import ctypes as C
import os
import re

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROOT = os.path.dirname(PKG)
LIB_PATH = os.path.join(PKG, "libsnd_scan.so")
HEADER = os.path.join(ROOT, "include", "snd_scan.h")

SND_F32, SND_F16, SND_BF16 = 0, 1, 2
SCHED_AUTO, SCHED_PLANE, SCHED_STRIPS, SCHED_BANDS, SCHED_WAVEFRONT = 0, 1, 2, 3, 4
DIR_TOPLEFT, DIR_CORNERS = 0, 1
i32, i64, vp = C.c_int32, C.c_int64, C.c_void_p


class Shape(C.Structure):
    _fields_ = [(n, i32) for n in ("batch", "dim", "nrows", "ncols", "dstate", "n_groups", "delta_dim", "in_dtype")]


class Plan(C.Structure):
    _fields_ = [("n_chunks_x", i32), ("n_chunks_y", i32), ("x_inner", i32), ("xv_inner", i32),
                ("x_elems", i64), ("x_sd_elems", i64), ("x_v_elems", i64), ("bwd_workspace_bytes", i64),
                ("fwd_workspace_bytes", i64), ("auto_schedule", i32), ("auto_bwd_jobs", i32),
                ("dC_skew_bytes", i64), ("wavefront_workspace", i32), ("reserved_", i32)]


class FwdParams(C.Structure):
    _fields_ = ([("shape", Shape), ("out_dtype", i32), ("delta_softplus", i32)] +
                [(n, vp) for n in ("u", "delta", "B", "C", "A", "D", "delta_bias", "A_decay", "out", "x", "x_v", "x_sd")] +
                [(n, i64) for n in ("u_batch_stride", "u_d_stride", "u_h_stride",
                                    "delta_batch_stride", "delta_d_stride", "delta_h_stride",
                                    "A_d_stride", "A_dstate_stride",
                                    "B_batch_stride", "B_group_stride", "B_dstate_stride", "B_h_stride",
                                    "C_batch_stride", "C_group_stride", "C_dstate_stride", "C_h_stride",
                                    "out_batch_stride", "out_d_stride", "out_h_stride")] +
                [("workspace", vp), ("workspace_bytes", i64), ("schedule", i32), ("directions", i32), ("u_shared", i32), ("merge", i32), ("merge_weights", vp)])


class BwdParams(C.Structure):
    _fields_ = ([("f", FwdParams), ("dout", vp), ("dout_dtype", i32)] +
                [(n, i64) for n in ("dout_batch_stride", "dout_d_stride", "dout_h_stride")] +
                [(n, vp) for n in ("du", "ddelta", "dA", "dB", "dC", "dD", "ddelta_bias", "dA_decay", "workspace")] +
                [("workspace_bytes", i64), ("dmerge", vp)])


def declared_symbols():
    """Every function include/snd_scan.h declares."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(snd_[a-z_]+)\s*\(", text)))


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libsnd_scan.so is not built: run python official-cross-scan_amd/build.py")
        _lib = C.CDLL(LIB_PATH)
        _lib.snd_version.restype = C.c_int
        _lib.snd_status_string.restype = C.c_char_p
        _lib.snd_status_string.argtypes = [C.c_int]
        _lib.snd_make_plan.argtypes = [C.POINTER(Shape), C.POINTER(Plan)]
        _lib.snd_fwd.argtypes = [C.POINTER(FwdParams), vp]
        _lib.snd_bwd.argtypes = [C.POINTER(BwdParams), vp]
        _lib.snd_bwd_static.argtypes = [C.POINTER(BwdParams), vp]
        _lib.snd_static_workspace_bytes.restype = C.c_int64
        _lib.snd_init.argtypes = [C.c_int]
        _lib.snd_workspace_error.argtypes = [vp, vp]
        _lib.snd_debug_set_spin_limit.argtypes = [C.c_int]
        _lib.snd_debug_set_spin_limit.restype = None
        _lib.snd_debug_set_strip_slots.argtypes = [C.c_int]
        _lib.snd_debug_set_strip_slots.restype = None
    return _lib


def _dt(t):
    import torch
    return {torch.float32: SND_F32, torch.float16: SND_F16, torch.bfloat16: SND_BF16}[t.dtype]


def make_shape(u, delta, A, B):
    """dim comes from A: u may be [batch, dim / n_groups, H, W] (shared by the groups, u_shared)."""
    return Shape(u.shape[0], A.shape[0], u.shape[2], u.shape[3], A.shape[1], B.shape[1], delta.shape[1], _dt(u))


def make_plan(shape):
    plan = Plan()
    st = lib().snd_make_plan(C.byref(shape), C.byref(plan))
    return st, plan


def _ptr(t):
    return None if t is None else t.data_ptr()


def _fill_fwd(fp, shape, u, delta, A, B, Cc, D, delta_bias, delta_softplus, A_decay, out, x, x_v, x_sd,
              schedule=SCHED_AUTO, directions=DIR_TOPLEFT):
    fp.shape = shape
    fp.schedule = schedule
    fp.directions = directions
    fp.u_shared = int(u.shape[1] != A.shape[0])
    fp.out_dtype = _dt(out) if out is not None else SND_F32
    fp.delta_softplus = int(bool(delta_softplus))
    fp.u, fp.delta, fp.B, fp.C, fp.A = _ptr(u), _ptr(delta), _ptr(B), _ptr(Cc), _ptr(A)
    fp.D, fp.delta_bias, fp.A_decay = _ptr(D), _ptr(delta_bias), _ptr(A_decay)
    fp.out, fp.x, fp.x_v, fp.x_sd = _ptr(out), _ptr(x), _ptr(x_v), _ptr(x_sd)
    fp.u_batch_stride, fp.u_d_stride, fp.u_h_stride = u.stride(0), u.stride(1), u.stride(2)
    fp.delta_batch_stride, fp.delta_d_stride, fp.delta_h_stride = delta.stride(0), delta.stride(1), delta.stride(2)
    fp.A_d_stride, fp.A_dstate_stride = A.stride(0), A.stride(1)
    fp.B_batch_stride, fp.B_group_stride, fp.B_dstate_stride, fp.B_h_stride = B.stride()[:4]
    fp.C_batch_stride, fp.C_group_stride, fp.C_dstate_stride, fp.C_h_stride = Cc.stride()[:4]
    if out is not None:
        fp.out_batch_stride, fp.out_d_stride, fp.out_h_stride = out.stride(0), out.stride(1), out.stride(2)


def check(st):
    if st != 0:
        raise RuntimeError("snd status %d: %s" % (st, lib().snd_status_string(st).decode()))


def _stream(stream):
    import torch
    return torch.cuda.current_stream().cuda_stream if stream is None else stream


def carve_pair(shape_a, shape_b, skew_bytes, device, zero=False):
    """Two fp32 tensors from one allocation, the second `skew_bytes` past the 2 MiB-rounded end of the first
    (snd_plan.dC_skew_bytes: dB and dC, accumulated at equal offsets at the same time, must not sit a multiple of
    2 MiB apart, which is where separate large allocations land)."""
    import math
    import torch
    na, nb = math.prod(shape_a), math.prod(shape_b)
    off = ((na * 4 + (2 << 20) - 1) // (2 << 20) * (2 << 20) + int(skew_bytes)) // 4
    buf = (torch.zeros if zero else torch.empty)(off + nb, device=device, dtype=torch.float32)
    return buf[:na].view(shape_a), buf[off:off + nb].view(shape_b)


class FwdCall:
    """Outputs, saved state and the filled snd_fwd_params of one forward; launch() only enqueues."""

    def __init__(self, u, delta, A, B, Cc, D=None, delta_bias=None, delta_softplus=False, out_float=True,
                 A_decay=None, save=True, schedule=SCHED_AUTO, directions=DIR_TOPLEFT, merge=False, merge_weights=None):
        import torch
        self.keep = (u, delta, A, B, Cc, D, delta_bias, A_decay, merge_weights)
        shape = make_shape(u, delta, A, B)
        st, plan = make_plan(shape)
        check(st)
        self.plan = plan
        Bt, Dm, N = u.shape[0], A.shape[0], A.shape[1]
        f32 = dict(device=u.device, dtype=torch.float32)
        if merge:                                # fused CrossMerge: one zero-filled fp32 channel per feature
            self.out = torch.zeros((Bt, Dm // B.shape[1], u.shape[2], u.shape[3]), **f32)
        else:
            self.out = torch.empty((Bt, Dm, u.shape[2], u.shape[3]), device=u.device, dtype=torch.float32 if out_float else u.dtype)
        self.x_v = torch.empty((Bt, Dm, N, plan.n_chunks_y, plan.xv_inner), **f32)
        self.x = torch.empty((Bt, Dm, N, plan.n_chunks_x, plan.x_inner), **f32) if save else None
        self.x_sd = torch.empty((Bt, Dm, N, plan.n_chunks_x, plan.x_inner), **f32) if save else None
        self.params = FwdParams()
        _fill_fwd(self.params, shape, u, delta, A, B, Cc, D, delta_bias, delta_softplus, A_decay, self.out,
                  self.x, self.x_v, self.x_sd, schedule, directions)
        self.params.merge, self.params.merge_weights = int(merge), _ptr(merge_weights)
        self.ws = torch.empty(plan.fwd_workspace_bytes // 4 + 4, **f32)
        self.params.workspace, self.params.workspace_bytes = self.ws.data_ptr(), plan.fwd_workspace_bytes

    def launch(self, stream=None):
        if self.params.merge:
            self.out.zero_()
        check(lib().snd_fwd(C.byref(self.params), _stream(stream)))


class BwdCall:
    """Gradient buffers, scratch and the filled snd_bwd_params of one backward.  launch() zero-fills
    the accumulated gradients (as the reference host does, selective_scan_oflex.cpp:395-403) and
    enqueues the kernel; launch_kernel_only() skips the zero-fill (timing)."""

    def __init__(self, u, delta, A, B, Cc, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd,
                 schedule=SCHED_AUTO, directions=DIR_TOPLEFT, merge=False, merge_weights=None):
        import torch
        self.keep = (u, delta, A, B, Cc, D, delta_bias, A_decay, dout, x, x_v, x_sd, merge_weights)
        shape = make_shape(u, delta, A, B)
        st, plan = make_plan(shape)
        check(st)
        Dm = A.shape[0]
        f32 = dict(device=u.device, dtype=torch.float32)
        self.du = torch.empty((u.shape[0], Dm, u.shape[2], u.shape[3]), device=u.device, dtype=u.dtype)
        self.ddelta = torch.empty_like(self.du)
        self.dA = torch.zeros_like(A)
        self.dB, self.dC = carve_pair(tuple(B.shape), tuple(Cc.shape), plan.dC_skew_bytes, u.device, zero=True)
        self.dD = torch.zeros_like(D) if D is not None else None
        self.dbias = torch.zeros(Dm, **f32) if delta_bias is not None else None
        self.ddec = torch.zeros_like(A_decay) if A_decay is not None else None
        self.dmerge = torch.zeros(Dm, **f32) if merge else None    # merge_weights * d merge_weights per channel
        self.ws = torch.empty(plan.bwd_workspace_bytes // 4 + 4, **f32)
        bp = self.params = BwdParams()
        _fill_fwd(bp.f, shape, u, delta, A, B, Cc, D, delta_bias, delta_softplus, A_decay, None, x, x_v, x_sd,
                  schedule, directions)
        bp.dout, bp.dout_dtype = dout.data_ptr(), _dt(dout)
        bp.dout_batch_stride, bp.dout_d_stride, bp.dout_h_stride = dout.stride(0), dout.stride(1), dout.stride(2)
        bp.du, bp.ddelta = self.du.data_ptr(), self.ddelta.data_ptr()
        bp.dA, bp.dB, bp.dC = self.dA.data_ptr(), self.dB.data_ptr(), self.dC.data_ptr()
        bp.dD, bp.ddelta_bias, bp.dA_decay = _ptr(self.dD), _ptr(self.dbias), _ptr(self.ddec)
        bp.workspace, bp.workspace_bytes = self.ws.data_ptr(), plan.bwd_workspace_bytes
        bp.f.merge, bp.f.merge_weights, bp.dmerge = int(merge), _ptr(merge_weights), _ptr(self.dmerge)

    def zero(self):
        for t in (self.dA, self.dB, self.dC, self.dD, self.dbias, self.ddec, self.dmerge):
            if t is not None:
                t.zero_()

    def launch_kernel_only(self, stream=None):
        check(lib().snd_bwd(C.byref(self.params), _stream(stream)))

    def launch_static(self, stream=None):
        """The same backward through snd_bwd_static: the library's own static scratch, no workspace passed."""
        self.zero()
        q = BwdParams.from_buffer_copy(self.params)
        q.workspace, q.workspace_bytes = None, 0
        check(lib().snd_bwd_static(C.byref(q), _stream(stream)))

    def launch(self, stream=None):
        self.zero()
        self.launch_kernel_only(stream)


def fwd(u, delta, A, B, Cc, D=None, delta_bias=None, delta_softplus=False, out_float=True, A_decay=None,
        save=True, stream=None, schedule=SCHED_AUTO, directions=DIR_TOPLEFT):
    """Reference operator `fwd` (selective_scan_oflex.cpp:179-187) through the C ABI."""
    call = FwdCall(u, delta, A, B, Cc, D, delta_bias, delta_softplus, out_float, A_decay, save, schedule, directions)
    call.launch(stream)
    return call.out, call.x, call.x_v, call.x_sd


def bwd(u, delta, A, B, Cc, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd, stream=None,
        schedule=SCHED_AUTO, directions=DIR_TOPLEFT):
    """Reference operator `bwd` (selective_scan_oflex.cpp:286-297, return list :432-438)."""
    call = BwdCall(u, delta, A, B, Cc, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd, schedule,
                   directions)
    call.launch_kernel_only(stream)
    Bt, _, H, W = u.shape
    Dm, Dd = A.shape[0], delta.shape[1]
    ddelta, dbias = call.ddelta, call.dbias
    du = call.du
    if u.shape[1] != Dm:                         # u shared by the groups: its gradient is the sum over them
        du = du.view(Bt, Dm // u.shape[1], u.shape[1], H, W).sum(1)
    if Dd != Dm:
        ddelta = ddelta.view(Bt, Dd, Dm // Dd, H, W).sum(2)
        if dbias is not None:
            dbias = dbias.view(Dd, Dm // Dd).sum(1)
    return du, ddelta, call.dA, call.dB.to(B.dtype), call.dC.to(Cc.dtype), call.dD, dbias, call.ddec
