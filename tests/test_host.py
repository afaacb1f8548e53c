"""CPU-only checks of the boundary: the C-ABI library loads, exports every symbol the header
declares, plans and validates like the reference's host code, and fails loudly without a GPU path."""
import ctypes as C
import os

import numpy as np
import pytest

import capi


def test_library_exports_every_declared_symbol():
    names = capi.declared_symbols()
    assert set(names) >= {"snd_version", "snd_status_string", "snd_make_plan", "snd_fwd", "snd_bwd", "snd_init",
                          "snd_workspace_error", "snd_debug_set_spin_limit", "snd_debug_set_strip_slots", "snd_bwd_static",
                          "snd_static_workspace_bytes"}
    lib = capi.lib()
    for n in names:
        assert getattr(lib, n) is not None, n
    assert lib.snd_version() >= 210


def test_struct_layouts_match_header_sizes():
    # field-by-field mirror of include/snd_scan.h: natural alignment, no packing
    assert C.sizeof(capi.Shape) == 32
    assert C.sizeof(capi.Plan) == 80
    assert C.sizeof(capi.FwdParams) == 32 + 8 + 12 * 8 + 19 * 8 + 8 + 8 + 4 * 4 + 8
    assert C.sizeof(capi.BwdParams) == C.sizeof(capi.FwdParams) + 8 + 8 + 3 * 8 + 9 * 8 + 8 + 8


def test_struct_layouts_match_the_c_compiler(tmp_path):
    """sizeof / offsetof of the header's structs as gcc sees them against the ctypes mirror."""
    import subprocess
    probes = [("snd_plan", capi.Plan, ["fwd_workspace_bytes", "bwd_workspace_bytes", "auto_schedule", "auto_bwd_jobs", "dC_skew_bytes", "wavefront_workspace"]),
              ("snd_fwd_params", capi.FwdParams, ["out", "x_sd", "u_batch_stride", "out_h_stride", "workspace", "schedule", "directions", "u_shared", "merge", "merge_weights"]),
              ("snd_bwd_params", capi.BwdParams, ["dout", "dout_dtype", "dout_batch_stride", "du", "workspace", "workspace_bytes", "dmerge"])]
    src = ["#include <stdio.h>", "#include <stddef.h>", '#include "snd_scan.h"', "int main(void) {"]
    for cname, _, fields in probes:
        src.append('printf("%%zu\\n", sizeof(%s));' % cname)
        for f in fields:
            src.append('printf("%%zu\\n", offsetof(%s, %s));' % (cname, f))
    src += ["return 0; }"]
    (tmp_path / "probe.c").write_text("\n".join(src))
    exe = str(tmp_path / "probe")
    subprocess.check_call(["gcc", "-I", os.path.join(capi.ROOT, "include"), str(tmp_path / "probe.c"), "-o", exe])
    got = [int(v) for v in subprocess.check_output([exe]).split()]
    want = []
    for _, cls, fields in probes:
        want.append(C.sizeof(cls))
        want += [getattr(cls, f).offset for f in fields]
    assert got == want


def test_placement_advice():
    """dC is to be carved past the 2 MiB-rounded end of dB by a multiple of 256 bytes that is no multiple of 2 MiB: half
    an fp32 row for the row-segment kernels on rows of 2 KiB or more."""
    for shp, want in (((64, 192, 56, 56, 16, 4, 192, capi.SND_F32), 5120), ((1, 256, 512, 512, 1, 4, 256, capi.SND_BF16), 1024),
                      ((1, 64, 1024, 1024, 1, 4, 64, capi.SND_BF16), 2048), ((8, 192, 64, 64, 1, 4, 192, capi.SND_BF16), 16384),
                      ((64, 768, 14, 14, 16, 4, 768, capi.SND_BF16), 5120)):
        st, plan = capi.make_plan(capi.Shape(*shp))
        assert st == 0
        assert plan.dC_skew_bytes == want
        assert plan.dC_skew_bytes % 256 == 0 and 0 < plan.dC_skew_bytes < (2 << 20)


@pytest.mark.parametrize("H,W,ncx,ncy", [(56, 56, 7, 7), (14, 14, 2, 2), (200, 336, 42, 25), (1, 37, 5, 1), (512, 512, 64, 64),
                                         (28, 28, 4, 4), (21, 35, 5, 3), (7, 7, 1, 1)])   # the last three use 7x7 tiles
def test_plan_geometry(H, W, ncx, ncy):
    st, plan = capi.make_plan(capi.Shape(2, 8, H, W, 16, 4, 8, capi.SND_F32))
    assert st == 0
    assert (plan.n_chunks_x, plan.n_chunks_y) == (ncx, ncy)
    assert plan.x_inner == ncy * 8 and plan.xv_inner == ncx * 8
    planes = 2 * 8 * 16
    assert plan.x_elems == planes * ncx * plan.x_inner == plan.x_sd_elems
    assert plan.x_v_elems == planes * ncy * plan.xv_inner
    sync_words = (12 + 2 * (2 * 4 * 1 * ncy) + 3) // 4 * 4   # header + two counters per (batch * groups * chunks) * strips
    assert plan.fwd_workspace_bytes == sync_words * 4 + planes * plan.xv_inner * 4
    assert plan.auto_schedule == (capi.SCHED_STRIPS if ncy > 1 else capi.SCHED_PLANE)   # 8 plane chunks only
    assert plan.bwd_workspace_bytes == sync_words * 4 + planes * plan.xv_inner * 4      # (8 plane chunks: no column segments)


@pytest.mark.parametrize("shape,code", [
    ((1, 6, 4, 4, 16, 4, 6, 0), -2),     # dim % n_groups != 0      (selective_scan_oflex.cpp:215)
    ((1, 8, 4, 4, 16, 4, 3, 0), -2),     # dim % delta_dim != 0     (:216)
    ((1, 8, 4, 4, 17, 4, 8, 0), -2),     # dstate > MAX_DSTATE      (:217)
    ((0, 8, 4, 4, 16, 4, 8, 0), -2),
    ((1, 8, 4, 4, 16, 4, 8, 7), -3),     # unknown dtype            (:190)
])
def test_plan_rejects_what_the_reference_rejects(shape, code):
    st, _ = capi.make_plan(capi.Shape(*shape))
    assert st == code
    assert len(capi.lib().snd_status_string(st)) > 0


def test_entry_points_validate_before_touching_the_gpu():
    lib = capi.lib()
    assert lib.snd_fwd(None, None) == -1
    assert lib.snd_bwd(None, None) == -1
    fp = capi.FwdParams()
    fp.shape = capi.Shape(1, 8, 4, 4, 16, 4, 8, capi.SND_F32)
    assert lib.snd_fwd(C.byref(fp), None) == -1            # null tensors
    fp.u = fp.delta = fp.A = fp.B = fp.C = 16
    assert lib.snd_fwd(C.byref(fp), None) == -6            # saved state missing
    fp.x_v = 24                                            # not 16-byte aligned
    assert lib.snd_fwd(C.byref(fp), None) == -7
    assert b"16-byte" in lib.snd_status_string(-7)


def test_address_range_limits_are_status_codes():
    """The kernels use unsigned 32-bit byte offsets inside a batch image and 24-bit row-pitch
    multiplies; shapes or strides beyond that are refused before anything is launched."""
    lib = capi.lib()

    def params(H=4, W=4, dim=8, **strides):
        fp = capi.FwdParams()
        fp.shape = capi.Shape(1, dim, H, W, 16, 4, dim, capi.SND_F32)
        fp.u = fp.delta = fp.A = fp.B = fp.C = fp.x_v = fp.out = 16
        fp.u_h_stride = fp.delta_h_stride = fp.B_h_stride = fp.C_h_stride = fp.out_h_stride = W
        fp.u_d_stride = fp.delta_d_stride = fp.out_d_stride = H * W
        fp.B_dstate_stride = fp.C_dstate_stride = H * W
        for k, v in strides.items():
            setattr(fp, k, v)
        return fp

    assert lib.snd_fwd(C.byref(params(schedule=9)), None) == -2                  # unknown schedule
    assert lib.snd_fwd(C.byref(params(schedule=capi.SCHED_STRIPS)), None) == -6  # pipelined schedules need the workspace
    assert lib.snd_fwd(C.byref(params(schedule=capi.SCHED_BANDS)), None) == -6
    assert lib.snd_fwd(C.byref(params(directions=2)), None) == -2                # unknown directions
    assert lib.snd_fwd(C.byref(params(u_h_stride=2)), None) == -4                # rows overlap
    assert lib.snd_fwd(C.byref(params(u_h_stride=1 << 21)), None) == -4          # row pitch >= 2^23 bytes
    assert lib.snd_fwd(C.byref(params(u_d_stride=1 << 28)), None) == -4          # image >= 2^32 bytes
    assert lib.snd_fwd(C.byref(params(out_d_stride=-1)), None) == -4             # negative stride
    assert lib.snd_fwd(C.byref(params(H=1 << 15, W=1 << 15, dim=8)), None) == -4  # dense gradients >= 2^32 bytes
    assert lib.snd_fwd(C.byref(params(H=1, W=1 << 21, dim=4)), None) == -4         # 2^21 columns: beyond the 24-bit column math
    assert lib.snd_fwd(C.byref(params(merge=2)), None) == -2                      # fused merge is a flag
    assert lib.snd_fwd(C.byref(params(merge=1, out_dtype=capi.SND_BF16)), None) == -3   # merged output is accumulated in fp32
    assert b"2^32" in lib.snd_status_string(-4)


def test_python_operator_has_no_cpu_fallback():
    torch = pytest.importorskip("torch")
    import selective_nd_scan as s
    with pytest.raises(RuntimeError, match="GPU"):
        s.selective_nd_scan(torch.zeros(1, 4, 3, 4), torch.zeros(1, 4, 3, 4), torch.zeros(4, 2),
                            torch.zeros(1, 1, 2, 3, 4), torch.zeros(1, 1, 2, 3, 4))


def test_extension_checks_mirror_reference_messages():
    torch = pytest.importorskip("torch")
    import selective_nd_scan as s
    z = torch.zeros
    with pytest.raises(RuntimeError):                       # A must be fp32 (:191)
        s.fwd(z(1, 4, 3, 4), z(1, 4, 3, 4), z(4, 2, dtype=torch.float16), z(1, 1, 2, 3, 4), z(1, 1, 2, 3, 4))
    with pytest.raises(RuntimeError):                       # dtype mismatch (:193)
        s.fwd(z(1, 4, 3, 4), z(1, 4, 3, 4, dtype=torch.float16), z(4, 2), z(1, 1, 2, 3, 4), z(1, 1, 2, 3, 4))


def test_cross_scan_host_helpers():
    """Direction-major layout helpers of the four-corner block (pure tensor bookkeeping, CPU)."""
    import torch
    import importlib
    cs = importlib.import_module("selective_nd_scan.cross_scan")   # the module, not the function of that name
    x = torch.arange(2 * 3 * 4 * 5, dtype=torch.float32).reshape(2, 3, 4, 5)
    xs = cs.cross_scan(x)
    assert xs.shape == (2, 12, 4, 5) and torch.equal(xs[:, 3:6], x) and torch.equal(xs[:, 9:], x)
    f = cs.flip_groups(xs, 4)
    assert torch.equal(f[:, 0:3], x) and torch.equal(f[:, 3:6], x.flip(-1))
    assert torch.equal(f[:, 6:9], x.flip(-2)) and torch.equal(f[:, 9:12], x.flip(-2, -1))
    assert torch.equal(cs.flip_groups(f, 4), xs)                       # an involution
    b5 = torch.randn(2, 8, 3, 4, 5)
    f5 = cs.flip_groups(b5, 8)
    assert torch.equal(f5[:, 5], b5[:, 5].flip(-1)) and torch.equal(cs.flip_groups(f5, 8), b5)
    assert torch.equal(cs.cross_merge(xs), 4 * x)
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    assert torch.allclose(cs.cross_merge(xs, w), 10 * x)
    wc = torch.arange(12, dtype=torch.float32).reshape(4, 3)
    assert torch.allclose(cs.cross_merge(xs, wc), x * wc.sum(0).reshape(1, 3, 1, 1))


def test_backward_job_split():
    """What AUTO gives the backward: whole planes, one job per strip (few plane chunks), or a few bands
    of strips when the plane chunks do not fill the chip's 512 block slots evenly."""
    def jobs(Bt, Dm, H, W, K=4):
        st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, 16, K, Dm, capi.SND_F32))
        assert st == 0
        return plan.auto_bwd_jobs, plan.n_chunks_y
    assert jobs(64, 192, 56, 56) == (2, 7)        # 768 plane chunks: two rounds, the second half empty -> two bands
    assert jobs(64, 768, 14, 14) == (0, 2)        # 3072 chunks = six full rounds
    assert jobs(2, 192, 200, 336) == (25, 25)     # 24 chunks: one job per strip
    assert jobs(1, 256, 512, 512) == (64, 64)
    assert jobs(43, 192, 56, 56) == (3, 7)        # 516 chunks: 4 rounds of a third instead of 2 whole ones
    assert jobs(64, 192, 8, 56) == (0, 1)         # a single strip cannot be split
    assert jobs(32, 192, 56, 56) == (7, 7)        # 384 chunks leave the chip short of waves: one job per strip
    assert jobs(40, 192, 56, 56) == (0, 7)        # 480 chunks are all resident at once: a plane's bands are a chain
    assert jobs(8, 768, 14, 14) == (0, 2)         # 384 chunks of two strips: nothing to run side by side
    assert jobs(85, 192, 56, 56) == (2, 7)        # 1020 chunks, but 129 of them pinned to each of four XCDs: 3 rounds
    assert jobs(128, 192, 56, 56) == (0, 7)       # 1536 chunks: three full rounds
    assert jobs(72, 192, 56, 56) == (2, 7)        # 864: the second round of whole planes would be 0.69 full and run at full-round pace
    assert jobs(80, 192, 56, 56) == (0, 7)        # 960: nearly two full rounds either way


def test_forward_job_split():
    """The forward holds 768 blocks at once (1536 with the 8-state kernels' smaller blocks)."""
    def sched(Bt, Dm, H, W, N=16, K=4):
        st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, N, K, Dm, capi.SND_F32))
        assert st == 0
        return plan.auto_schedule
    assert sched(64, 192, 56, 56) == capi.SCHED_PLANE     # 768 plane chunks on 768 slots
    assert sched(70, 192, 56, 56) == capi.SCHED_BANDS     # 840: a second round for 72 blocks otherwise
    assert sched(128, 192, 56, 56) == capi.SCHED_PLANE    # 1536: two full rounds
    assert sched(70, 192, 56, 56, N=8) == capi.SCHED_STRIPS  # 840 chunks, between the backward's 768 slots and 0.8 x 1536 (measured 0.45 against 0.51 ms)
    assert sched(64, 192, 56, 56, N=8) == capi.SCHED_STRIPS  # the 8-state forward prefers strips up to one full round of wide planes
    assert sched(128, 192, 56, 56, N=8) == capi.SCHED_STRIPS # 1536 of 1536 slots (measured 0.70 against 0.83 ms)
    assert sched(256, 192, 56, 56, N=8) == capi.SCHED_PLANE  # two full rounds
    assert sched(64, 768, 14, 14, N=8) == capi.SCHED_PLANE   # 2 x 2 tiles: nothing to run side by side
    assert sched(48, 192, 56, 56) == capi.SCHED_STRIPS    # 576 chunks: whole planes would put a third block on a quarter of the CUs
    assert sched(56, 192, 56, 56) == capi.SCHED_PLANE     # 672: beyond 0.8 x 768
    assert sched(112, 192, 56, 56) == capi.SCHED_BANDS    # 1344: 1.75 rounds
    assert sched(2, 192, 200, 336) == capi.SCHED_STRIPS
    assert sched(24, 192, 56, 56) == capi.SCHED_STRIPS    # 288 plane chunks: strips fill the chip better
    assert sched(40, 192, 56, 56) == capi.SCHED_PLANE
    assert sched(70, 192, 8, 56) == capi.SCHED_PLANE      # one strip


def test_kernel_family_choice():
    """1-4 states: the row-segment wavefront (narrow planes packed two or four to a wave), except for a few plane
    sizes with four states where a wave's lanes stay too empty; 5-16 states always the tile kernels."""
    def family(Bt, Dm, H, W, N, K=4):
        st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, N, K, Dm, capi.SND_BF16))
        assert st == 0
        assert plan.auto_bwd_jobs == 0 or plan.auto_schedule != capi.SCHED_WAVEFRONT
        return "wave" if plan.auto_schedule == capi.SCHED_WAVEFRONT else "tile"
    assert family(1, 256, 512, 512, 1) == "wave"          # 256 planes: nothing else fills the chip
    assert family(64, 192, 56, 56, 1) == "wave"
    assert family(64, 384, 28, 28, 1) == "wave"
    assert family(64, 768, 14, 14, 1) == "wave"           # four planes per wave
    assert family(64, 1536, 7, 7, 1) == "wave"
    assert family(64, 768, 14, 14, 4) == "wave"
    assert family(32, 12288, 7, 7, 4) == "wave"           # eight planes per wave: 0.59 ms against 0.65
    assert family(32, 1344, 21, 21, 4) == "wave"          # (0.66 against 0.67)
    assert family(32, 256, 40, 40, 4) == "tile"
    assert family(64, 192, 56, 56, 4) == "wave"           # (the two families within 2 % of each other)
    assert family(4, 192, 56, 56, 4) == "wave"            # 48 blocks: the strip pipeline's ramp costs more than the rows
    assert family(64, 192, 56, 56, 2) == "wave"
    assert family(64, 192, 56, 56, 16) == "tile"
    assert family(1, 8, 9, 1500, 4, K=2) == "wave"         # a wide plane: 24 row segments in three column groups
    assert family(2, 64, 256, 1024, 2) == "wave"
    assert family(1, 8, 9, 1500, 5, K=2) == "tile"


def test_wide_plane_plan():
    """More than eight row segments: the row-segment kernels take the plane in column groups that hand over through
    memory - the plan says so and sizes both workspaces for it; narrower planes need none."""
    def plan_of(H, W, N, Bt=1, Dm=8):
        st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, N, 2, Dm, capi.SND_F32))
        assert st == 0
        return plan
    assert plan_of(9, 512, 2).wavefront_workspace == 0
    assert plan_of(9, 1024, 1).wavefront_workspace == 0     # one state, even width: two columns per lane, eight segments
    assert plan_of(9, 1023, 1).wavefront_workspace == 1     # odd: one column per lane, 16 segments
    assert plan_of(9, 513, 2).wavefront_workspace == 1
    assert plan_of(9, 2048, 16).wavefront_workspace == 0    # (5-16 states: the tile kernels)
    p = plan_of(10, 1500, 2)
    planes, Hp, nseg, groups = 8 * 2, 10, 24, 3
    assert p.wavefront_workspace == 1
    assert p.x_elems >= planes * nseg * 2 * Hp              # column checkpoints of all 24 segments
    assert p.bwd_workspace_bytes >= planes * groups * 3 * Hp * 4
    assert p.fwd_workspace_bytes >= 2 * planes * nseg * 2 * Hp * 4


def test_split_plane_plan():
    """Few planes of eight row segments with one or two states: the backward may cut them in two halves that hand over
    through tagged words in the workspace - the plan says so and sizes the backward's workspace for the words."""
    def plan_of(Bt, Dm, H, W, N):
        st, plan = capi.make_plan(capi.Shape(Bt, Dm, H, W, N, 4, Dm, capi.SND_BF16))
        assert st == 0
        return plan
    p = plan_of(1, 256, 512, 512, 1)                        # 256 planes x 8 segments
    assert p.auto_schedule == capi.SCHED_WAVEFRONT and p.wavefront_workspace == 1
    assert p.bwd_workspace_bytes >= 256 * (512 // 4) * 3 * 4 * 8     # planes x bands x (G, Gs, a) x rows per band x 8 bytes
    assert plan_of(1, 256, 512, 512, 2).wavefront_workspace == 1
    assert plan_of(1, 256, 512, 512, 4).wavefront_workspace == 0    # three and four states: whole planes
    assert plan_of(1, 256, 512, 384, 1).wavefront_workspace == 0    # six segments: whole planes
    assert plan_of(2, 256, 512, 512, 1).wavefront_workspace == 0    # 512 planes: two channels share a block of 16 waves
    assert plan_of(1, 64, 512, 512, 1).wavefront_workspace == 0     # 512 waves: too few to be worth the pairing


def test_tile_extent_choice():
    """7x7 tiles where they leave clearly fewer padded cells (the 14 / 28 / 7 stage sizes), else 8x8."""
    def tiles(H, W):
        st, plan = capi.make_plan(capi.Shape(1, 4, H, W, 16, 1, 4, capi.SND_F32))
        assert st == 0
        return plan.n_chunks_y, plan.n_chunks_x
    assert tiles(14, 14) == (2, 2) and tiles(28, 28) == (4, 4) and tiles(7, 7) == (1, 1) and tiles(21, 35) == (3, 5)
    assert tiles(56, 56) == (7, 7) and tiles(64, 64) == (8, 8) and tiles(512, 512) == (64, 64) and tiles(200, 336) == (25, 42)
    assert tiles(1, 37) == (1, 5)                 # 294 vs 320 padded cells: not worth the smaller tile


def test_static_workspace_entry_point_validates_on_the_host():
    """snd_bwd_static refuses bad calls before it touches a GPU: null parameters, bad shapes, and shapes
    whose scratch does not fit the static workspace (with the status code and text that say so)."""
    lib = capi.lib()
    limit = lib.snd_static_workspace_bytes()
    assert limit == 64 << 20
    assert lib.snd_bwd_static(None, None) == -1
    bp = capi.BwdParams()
    bp.f.shape = capi.Shape(1, 6, 4, 4, 16, 4, 6, capi.SND_F32)          # dim % n_groups != 0
    assert lib.snd_bwd_static(C.byref(bp), None) == -2
    big = capi.Shape(64, 768, 56, 56, 16, 4, 768, capi.SND_F32)          # needs 176 MB of adjoint rows
    st, plan = capi.make_plan(big)
    assert st == 0 and plan.bwd_workspace_bytes > limit
    bp.f.shape = big
    assert lib.snd_bwd_static(C.byref(bp), None) == -8
    assert b"static workspace" in lib.snd_status_string(-8)
    for cfg in [(64, 192, 56, 56, 16, 4), (64, 768, 14, 14, 16, 4), (2, 192, 200, 336, 16, 4), (1, 256, 512, 512, 16, 4)]:
        st, plan = capi.make_plan(capi.Shape(*cfg, cfg[1], capi.SND_F32))
        assert st == 0 and plan.bwd_workspace_bytes <= limit, cfg        # every benchmark configuration fits


def test_pipeline_error_contract_on_the_host():
    """The documented error query and status text exist and validate their arguments; the spin-limit
    hook accepts any value (<= 0 restores the default)."""
    lib = capi.lib()
    assert lib.snd_workspace_error(None, None) == -1
    assert b"timed out" in lib.snd_status_string(-9) and b"NaN" in lib.snd_status_string(-9)
    lib.snd_debug_set_spin_limit(3)
    lib.snd_debug_set_spin_limit(0)
    header = open(capi.HEADER).read()
    assert "word [1] is an error flag" in header and "snd_workspace_error" in header


def test_init_without_a_gpu_is_a_status_not_a_crash():
    torch = pytest.importorskip("torch")
    if torch.cuda.is_available():
        pytest.skip("needs a box without a GPU")
    assert capi.lib().snd_init(0) == -5


def test_reference_module_name_is_importable():
    """Callers of the reference `import selective_nd_scan_cuda_oflex` (setup.py:80): the same name here is
    the gfx950 extension, with the reference's two functions."""
    pytest.importorskip("torch")
    import selective_nd_scan_cuda_oflex as m
    import selective_nd_scan_hip_oflex as h
    assert m.fwd is h.fwd and m.bwd is h.bwd
    assert "schedule" in m.fwd.__doc__ and "directions" in m.bwd.__doc__


def test_packaging_names_match_the_reference():
    """setup.py: distribution `selective_nd_scan` (reference setup.py:118), extension module
    `selective_nd_scan_cuda_oflex` (:80)."""
    text = open(os.path.join(capi.ROOT, "setup.py")).read()
    assert 'name="selective_nd_scan"' in text and '"selective_nd_scan_cuda_oflex"' in text


def test_plan_sizes_the_backward_workspace_for_column_segments():
    """More strip jobs than the backward's block slots: the strips are cut into column segments, whose carried column
    state (one slot of 13 x 2 x 256 floats per strip) the plan adds to the backward's workspace."""
    st, plan = capi.make_plan(capi.Shape(2, 192, 200, 336, 16, 4, 192, capi.SND_F32))     # 24 plane chunks x 25 strips on 512 slots
    assert st == 0 and plan.auto_schedule == capi.SCHED_STRIPS
    planes, chunks = 2 * 192 * 16, 24
    sync_words = (12 + 2 * chunks * 25 + 3) // 4 * 4
    assert plan.fwd_workspace_bytes == sync_words * 4 + planes * plan.xv_inner * 4
    assert plan.bwd_workspace_bytes == plan.fwd_workspace_bytes + chunks * 25 * 13 * 2 * 256 * 4
    st, plan = capi.make_plan(capi.Shape(1, 256, 512, 512, 16, 4, 256, capi.SND_BF16))    # 1024 strips of 64 tiles: nothing to gain
    assert st == 0 and plan.bwd_workspace_bytes == plan.fwd_workspace_bytes
