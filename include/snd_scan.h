/*
 * snd_scan.h — C ABI of the MI355X (gfx950) 2D-CrossScan selective scan, forward and backward.
 *
 * This is the drop-in boundary for the reference's one operator pair
 *     fwd(u, delta, A, B, C, D, delta_bias, delta_softplus, out_float, A_decay) -> [out, x, x_v, x_sd]
 *     bwd(u, delta, A, B, C, D, delta_bias, dout, x, x_v, delta_softplus, A_decay, x_sd)
 *         -> [du, ddelta, dA, dB, dC, dD, ddelta_bias, dA_decay]
 * (reference: kernels/selective_nd_scan/src/cusoflex/selective_scan_oflex.cpp:179-187,286-297,442-445).
 *
 * Plain pointers and sizes only.  The library never allocates device memory, never synchronises
 * and never throws: every entry point returns an int status (0 = ok, negative = error) and
 * enqueues its work on the HIP stream it is given.  The caller (the PyTorch extension, or any
 * other host) validates ownership, allocates outputs / checkpoints / workspace and passes them in.
 *
 * Tensor layouts are the reference's (selective_scan_oflex.cpp:206-229):
 *     u      [batch, dim, nrows, ncols]            input dtype, last dim contiguous
 *     delta  [batch, delta_dim, nrows, ncols]      input dtype, last dim contiguous
 *     A      [dim, dstate]                         fp32
 *     B, C   [batch, n_groups, dstate, nrows, ncols] input dtype, last dim contiguous
 *     D      [dim] fp32 (optional), delta_bias [delta_dim] fp32 (optional), A_decay [1] fp32 (optional)
 *     out    [batch, dim, nrows, ncols]            fp32 or input dtype
 * dim % n_groups == 0, dim % delta_dim == 0, dstate <= 16.  All strides are in ELEMENTS.
 */
#ifndef SND_SCAN_H
#define SND_SCAN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SND_MAX_DSTATE 16          /* selective_scan_common.h:13 (MAX_DSTATE) */

typedef void *snd_stream_t;        /* a hipStream_t, passed opaquely */

typedef enum snd_dtype { SND_F32 = 0, SND_F16 = 1, SND_BF16 = 2 } snd_dtype;

typedef enum snd_status {
    SND_OK = 0,
    SND_ERR_NULL = -1,             /* a required pointer is null */
    SND_ERR_SHAPE = -2,            /* sizes violate the reference's checks (host.cpp:215-245) */
    SND_ERR_DTYPE = -3,            /* unsupported dtype combination (host.cpp:190-195) */
    SND_ERR_STRIDE = -4,           /* a stride is negative / zero where a dense walk is required */
    SND_ERR_LAUNCH = -5,           /* hipLaunchKernel reported an error */
    SND_ERR_WORKSPACE = -6,        /* checkpoint / workspace buffer missing or too small */
    SND_ERR_ALIGN = -7,            /* checkpoint / workspace pointer not 16-byte aligned */
    SND_ERR_TOO_LARGE = -8,        /* snd_bwd_static: the shape needs more scratch than the static workspace holds */
    SND_ERR_PIPELINE = -9          /* snd_workspace_error: a hand-over wait between blocks timed out (outputs are NaN) */
} snd_status;

/* Problem sizes; replaces the size fields of SSMParamsBase
 * (kernels/selective_nd_scan/include/cusoflex/selective_scan_oflex.h:4-20). */
typedef struct snd_shape {
    int32_t batch, dim, nrows, ncols, dstate, n_groups, delta_dim;
    int32_t in_dtype;              /* snd_dtype of u, delta, B, C */
} snd_shape;

/* Sizes (in fp32 elements) of the opaque state that fwd hands to bwd and of bwd's scratch.
 * Replaces the nChunksX / nChunksY arithmetic and the three torch::empty calls of
 * selective_scan_oflex.cpp:247-258.  The tensors keep the reference's ranks so that call sites
 * written for the reference still work:
 *     x     [batch, dim, dstate, n_chunks_x, x_inner]     (h at the right edge of every column tile)
 *     x_sd  [batch, dim, dstate, n_chunks_x, x_inner]     (row-only scan s at the same places)
 *     x_v   [batch, dim, dstate, n_chunks_y, xv_inner]    (h at the last row of every row strip)
 * (sized so that either kernel family fits where both apply).
 * Their contents are private to this library; bwd does NOT modify them (a second backward over
 * the same saved state is valid, unlike the reference, bwd.cuh:489-491,614-619,725-727). */
typedef struct snd_plan {
    int32_t n_chunks_x, n_chunks_y;
    int32_t x_inner, xv_inner;
    int64_t x_elems, x_sd_elems, x_v_elems;    /* fp32 element counts of the three tensors */
    int64_t bwd_workspace_bytes;               /* scratch bwd needs (16-byte aligned, uninitialised) */
    int64_t fwd_workspace_bytes;               /* scratch fwd uses when it splits planes into strips
                                                  (16-byte aligned, uninitialised; one row per plane) */
    int32_t auto_schedule;                     /* what SND_SCHED_AUTO resolves to in the forward for this shape
                                                  (PLANE, STRIPS, BANDS or WAVEFRONT): a caller may skip the fwd
                                                  workspace for PLANE and WAVEFRONT (see wavefront_workspace) */
    int32_t auto_bwd_jobs;                     /* jobs per plane chunk SND_SCHED_AUTO gives the backward: 0 = one
                                                  block per plane chunk (also when auto_schedule is WAVEFRONT: then
                                                  the backward runs WAVEFRONT too and needs no workspace unless
                                                  wavefront_workspace is 1),
                                                  n_chunks_y = one per strip, 2-4 = bands */
    /* Placement advice for callers that allocate the buffers (no counterpart in the reference, which leaves
     * placement to torch::empty).  The backward accumulates dB and dC at equal offsets at the same time.
     * Separate large allocations start 2 MiB apart or a multiple of it, which on an MI355X puts the two
     * atomics of a pixel in the same memory bank: the row-segment backward at 256 planes of 512x512, N=1 takes
     * 0.55-0.63 ms that way and 0.46-0.50 ms with dC half an fp32 row further on.  Put both in one allocation,
     * dC at dB + round_up(bytes of dB, 2 MiB) + dC_skew_bytes (a multiple of 256; the distance the advice was
     * measured at).  Results do not depend on placement, and no other pair of buffers shows the effect
     * (timed with dC moved step by step inside one large allocation). */
    int64_t dC_skew_bytes;
    int32_t wavefront_workspace;               /* 1 if WAVEFRONT uses the workspace for this shape.  Planes taken in
                                                  column groups (rows of more than 512 columns; with one state and an
                                                  even width, more than 1024) hand over through memory: bwd then needs
                                                  its workspace (bwd_workspace_bytes covers it), and a fwd that saves
                                                  no state (x == NULL) needs fwd_workspace_bytes, or AUTO runs the tile
                                                  kernels.  Few planes of 449-512 columns with one or two
                                                  states (at most 256 planes, e.g. 256 of 512x512): bwd cuts each plane
                                                  in two halves that run side by side if it is given its workspace
                                                  (about a fifth faster), and runs whole planes without one */
    int32_t reserved_;
} snd_plan;

/* How a launch maps work to blocks.  The reference has one fixed mapping (one block per
 * (batch, channel), fwd.cuh:359-392); here the library picks by shape unless told otherwise:
 *   PLANE   one block per (batch, group, 16-channel chunk) walks the whole plane;
 *   STRIPS  one block per 8-row strip of such a chunk, the strips of a plane pipelined one tile
 *           apart (for few, large planes, e.g. 2 x 192 channels of 200x336 or 256 of 512x512).  Needs the workspace.
 *   BANDS   one block per band of consecutive strips, 2-4 bands per plane, handed over like strips but
 *           only at band ends.  For more plane chunks than the chip holds blocks at once (backward at B=64, D=192, 56x56, N=16:
 *           768 chunks, 512 slots), where whole-plane blocks leave the last round half empty.  Needs
 *           the workspace.
 *   WAVEFRONT  the second kernel family, for 1-4 states per channel: a block per (batch, channel), a wave
 *           per 64-column row segment, the segments of a plane advancing as an anti-diagonal wavefront
 *           (what AUTO picks whenever its timing model prefers it).  Planes of more than eight segments
 *           are taken in column groups of eight, one launch per group (snd_plan.wavefront_workspace).  Its saved state has a
 *           layout of its own: fwd and bwd of one call pair must both run WAVEFRONT or both run one of the
 *           three tile schedules above (AUTO decides by shape alone, so AUTO on both sides always agrees). */
typedef enum snd_schedule { SND_SCHED_AUTO = 0, SND_SCHED_PLANE = 1, SND_SCHED_STRIPS = 2, SND_SCHED_BANDS = 3, SND_SCHED_WAVEFRONT = 4 } snd_schedule;

/* Scan origin per group.  The reference scans every group from the top-left corner and leaves the
 * per-group order as a TODO (fwd.cuh:140); its callers build the four corner directions of the
 * 2D-CrossScan block by flipping copies of the inputs and un-flipping the outputs.
 *   TOPLEFT  every group runs top-left -> bottom-right (the reference's behaviour);
 *   CORNERS  group g starts at corner g % 4: 0 top-left, 1 top-right (columns reversed),
 *            2 bottom-left (rows reversed), 3 bottom-right (both).  All tensors stay in their natural
 *            orientation in memory: the result equals flipping u, delta, B, C of that group, scanning
 *            top-left, and flipping out (and every per-pixel gradient) back. */
typedef enum snd_directions { SND_DIR_TOPLEFT = 0, SND_DIR_CORNERS = 1 } snd_directions;

/* Replaces SSMParamsBase (selective_scan_oflex.h:4-51); 64-bit strides instead of uint32. */
typedef struct snd_fwd_params {
    snd_shape shape;
    int32_t out_dtype;             /* SND_F32 or shape.in_dtype (host.cpp:250, out_float) */
    int32_t delta_softplus;        /* host.cpp:184 */
    const void *u, *delta, *B, *C;
    const float *A;
    const float *D;                /* optional (null: D = 0, fwd.cuh:121-124) */
    const float *delta_bias;       /* optional (null: 0, fwd.cuh:125-128) */
    const float *A_decay;          /* optional, 1 element, must be > 0 (null: 1.0, fwd.cuh:131-134) */
    void *out;
    float *x, *x_v, *x_sd;         /* saved state sized by snd_make_plan, 16-byte aligned.  x_v is always
                                      required (it also carries h from one row strip to the next);
                                      x and x_sd may both be null = inference only (bwd impossible) */
    int64_t u_batch_stride, u_d_stride, u_h_stride;
    int64_t delta_batch_stride, delta_d_stride, delta_h_stride;
    int64_t A_d_stride, A_dstate_stride;
    int64_t B_batch_stride, B_group_stride, B_dstate_stride, B_h_stride;
    int64_t C_batch_stride, C_group_stride, C_dstate_stride, C_h_stride;
    int64_t out_batch_stride, out_d_stride, out_h_stride;
    void *workspace;               /* plan.fwd_workspace_bytes bytes, 16-byte aligned, or null (then the
                                      PLANE schedule is used).  In snd_bwd_params.f it is ignored. */
    int64_t workspace_bytes;
    int32_t schedule;              /* snd_schedule, for fwd and (through snd_bwd_params.f) for bwd */
    int32_t directions;            /* snd_directions, for fwd and (through snd_bwd_params.f) for bwd */
    int32_t u_shared;              /* 0: u is [batch, dim, nrows, ncols] (the reference's layout).
                                      1: u is [batch, dim / n_groups, nrows, ncols] and every group scans
                                      the same channels (channel g*(dim/n_groups) + i reads u channel i):
                                      the CrossScan of one feature map without its n_groups copies.
                                      out, du and every other tensor keep their dim-wide layouts. */
    int32_t merge;                 /* 0: out is [batch, dim, nrows, ncols] (the reference's layout).
                                      1: CrossMerge fused into the output stores: out is fp32
                                      [batch, dim / n_groups, nrows, ncols], zero-filled by the caller, and
                                      channel g*(dim/n_groups) + i adds merge_weights[that channel] * (its result)
                                      to out channel i with a float atomic, so out ends as the weighted sum of
                                      the n_groups results per feature (the summation order, hence the last
                                      bits, vary from run to run).  out_dtype must be SND_F32; out strides
                                      describe the merged tensor.  In snd_bwd_params.f it says that dout has
                                      the merged shape (see there).  No counterpart in the reference kernel:
                                      it is the fusion "with trainable weights" of README.md:45. */
    const float *merge_weights;    /* [dim] fp32, one weight per (group, feature) in channel order, or null
                                      (all ones: the plain CrossMerge sum).  Read only when merge = 1. */
} snd_fwd_params;

/* Replaces SSMParamsBwd (selective_scan_oflex.h:53-86). Gradient buffers are dense (contiguous):
 *     du      [batch, dim, nrows, ncols]          input dtype
 *     ddelta  [batch, dim, nrows, ncols]          input dtype, PER CHANNEL (dim, not delta_dim):
 *                                                 the caller sums channel groups when
 *                                                 dim != delta_dim, as host.cpp:433-434 does
 *     dA      [dim, dstate] fp32, accumulated with atomics: caller zero-fills (host.cpp:395)
 *     dB, dC  [batch, n_groups, dstate, nrows, ncols] fp32, accumulated with atomics: caller
 *                                                 zero-fills, then casts to the input dtype
 *                                                 (host.cpp:398-399,432)
 *     dD [dim], ddelta_bias [dim] (per channel, host.cpp:403), dA_decay [1]: fp32, optional,
 *                                                 accumulated with atomics: caller zero-fills
 * With f.merge = 1 (fused CrossMerge) dout is the gradient of the merged output,
 * [batch, dim / n_groups, nrows, ncols] with the dout strides describing that tensor; channel
 * g*(dim/n_groups) + i reads dout channel i scaled by merge_weights[g*(dim/n_groups) + i]. */
typedef struct snd_bwd_params {
    snd_fwd_params f;              /* inputs and saved state; f.out / f.out_dtype are ignored */
    const void *dout;              /* [batch, dim, nrows, ncols] (merged shape if f.merge), last dim contiguous */
    int32_t dout_dtype;            /* SND_F32 or shape.in_dtype (host.cpp:303) */
    int64_t dout_batch_stride, dout_d_stride, dout_h_stride;
    void *du, *ddelta;
    float *dA, *dB, *dC;
    float *dD, *ddelta_bias, *dA_decay;
    void *workspace;               /* plan.bwd_workspace_bytes bytes, 16-byte aligned */
    int64_t workspace_bytes;
    float *dmerge;                 /* [dim] fp32, optional, accumulated with atomics: caller zero-fills.
                                      With f.merge = 1 channel c receives
                                          merge_weights[c] * d loss / d merge_weights[c]
                                        = sum over batch and pixels of  merge_weights[c] * dout * (result of channel c)
                                      (every gradient of the op is linear in the weighted dout, so the kernel
                                      carries the weight through; the caller divides by merge_weights[c], and
                                      handles a weight of exactly 0 on the unfused path).  Ignored when
                                      f.merge = 0. */
} snd_bwd_params;

/* Library / ABI version (major*100 + minor). */
int snd_version(void);

/* Human-readable text for a status code. */
const char *snd_status_string(int status);

/* Validate a shape the way selective_scan_oflex.cpp:215-217 does and size the saved state and
 * backward scratch.  Returns SND_OK or SND_ERR_SHAPE / SND_ERR_DTYPE. */
int snd_make_plan(const snd_shape *shape, snd_plan *plan);

/* Forward: replaces selective_scan_fwd_cuda<input_t, weight_t, output_t>(params, stream)
 * (selective_scan_oflex.cpp:31-32,275-281; kernel fwd.cuh:80-357).  Asynchronous on `stream`. */
int snd_fwd(const snd_fwd_params *params, snd_stream_t stream);

/* Backward: replaces selective_scan_bwd_cuda<input_t, weight_t, output_t>(params, stream)
 * (selective_scan_oflex.cpp:34-35,424-430; kernel bwd.cuh:91-902).  Asynchronous on `stream`. */
int snd_bwd(const snd_bwd_params *params, snd_stream_t stream);

/* Per-device set-up: raises the dynamic-LDS limit of the backward kernels and looks up the static
 * workspace on `device` (replaces the cudaFuncSetAttribute calls the reference makes inside every launch,
 * bwd.cuh:913-915, fwd.cuh:368-370).  Optional: the first snd_bwd / snd_bwd_static on a device does the same,
 * but these runtime calls are not stream-ordered, so a host that captures launches into a HIP graph, or
 * launches from several threads at once, calls snd_init(device) once beforehand.  Thread-safe. */
int snd_init(int device);

/* The pipelined schedules (STRIPS, BANDS; what the plan's auto_schedule / auto_bwd_jobs say AUTO picks)
 * hand rows from block to block through the workspace.  Its first 12 int32 words are the launch's sync
 * header, cleared by the launch itself: word [1] is an error flag that a block sets when a wait for another
 * block's row exceeds its poll limit (2^21 polls: a stalled producer, e.g. on a preempted GPU).  Such a
 * block replaces the missing row by NaN, so out / du / ddelta / dA / dB / dC downstream of it are NaN,
 * never plausible numbers, and the launch still drains.  snd_fwd / snd_bwd have returned SND_OK long
 * before; this call is how a host learns the reason: it copies word [1] back and WAITS for `stream`
 * (the only synchronising call of the library).  Returns SND_OK, SND_ERR_PIPELINE, or another error.
 * Meaningful only after a pipelined launch on that workspace (a whole-plane launch leaves the header
 * alone).  workspace == NULL asks about the static scratch of snd_bwd_static on the current device.
 * No counterpart in the reference, whose blocks never wait for each other. */
int snd_workspace_error(const void *workspace, snd_stream_t stream);

/* Test hook: poll limit of the hand-over waits for later launches (<= 0 restores the default 2^21).
 * With a limit of a few polls the time-out path above can be exercised from the host while every
 * kernel still runs to completion. */
void snd_debug_set_spin_limit(int polls);

/* Test hook: the number of block slots the backward's strip-pipeline model assumes when it decides whether to cut
 * strips into column segments (0 restores the machine's own count); a negative value -n skips the model and cuts
 * every pipelined strip into n segments (at least two tiles each).  Small test shapes then take the segmented
 * path - plan sizes and launches alike - that only shapes with more strips than slots take otherwise. */
void snd_debug_set_strip_slots(int slots);

/* snd_bwd for callers that cannot allocate device memory (code under HIP-graph capture, serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference, which allocates its scratch with
 * torch::empty / torch::zeros inside every call (selective_scan_oflex.cpp:393-403).  Identical to
 * snd_bwd except that params->workspace / workspace_bytes are ignored: the scratch is a static device
 * array of snd_static_workspace_bytes() bytes (64 MiB per GPU, held until the process ends) that the
 * library owns.  Shapes whose plan.bwd_workspace_bytes exceeds it are refused with SND_ERR_TOO_LARGE (calls that
 * run the row-segment kernels use no scratch and are never refused for size).  A timed-out hand-over is reported
 * by snd_workspace_error(NULL, stream).
 * The caller still passes every input, output and saved-state buffer.  Allocates nothing, frees nothing.
 * All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race;
 * calls on one stream are ordered.  The sync header is cleared by a fill kernel at the start of each
 * launch; nothing else in the array needs to start at zero. */
int snd_bwd_static(const snd_bwd_params *params, snd_stream_t stream);
int64_t snd_static_workspace_bytes(void);

#ifdef __cplusplus
}
#endif
#endif /* SND_SCAN_H */
