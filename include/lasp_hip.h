/*
 * lasp_hip.h -- C ABI of liblasp_hip.so (gfx950 / MI355X).
 *
 * Causal decayed linear attention ("lightning attention") on one chunk of a
 * sequence, forward and backward, with an optional d x e fp32 state arriving
 * from the previous chunk (KV) and, in backward, from the next chunk (DKV).
 *
 * Tensor contract (all pointers are DEVICE pointers, all tensors contiguous,
 * row-major):
 *     q, k, dq, dk : (b, h, n, d)      element type `dtype`
 *     v, o, do, dv : (b, h, n, e)      element type `dtype`
 *     s            : h floats          per-head decay slope, >= 0
 *     kv_in, kv_out, dkv_in, dkv_out : (b, h, d, e) float, may be NULL
 *     seg states   : float workspace of lasp_plan's state_bytes (one state per (b, h) and segment, or per
 *                    piece of a long segment; each d x e, or zero-extended to 128 x 128): opaque to the caller
 *
 * Alignment: q, k, v, o, do, dq, dk, dv start on a 16-byte boundary (the kernels
 * fetch rows with 8- and 16-byte loads and store them with 16-byte stores; rows of d or e
 * 16-bit elements with d, e multiples of 8 keep every row aligned as well); s, the
 * states and the workspaces on a 4-byte boundary.  A pointer that is not returns
 * LASP_E_ALIGN.
 * Device: the calling thread's current device (hipSetDevice) must be the one that
 * owns every pointer and `stream`; the calls check this for q (LASP_E_DEVICE) and
 * never switch devices themselves.
 * Range: the 16-bit kernels round the fp32 states, the decayed keys and the masked
 * q.k scores to the I/O element type before each matrix product (accumulation is
 * fp32).  With fp16 I/O any of them beyond 65504 in magnitude becomes inf -- a large
 * caller-supplied kv_in, or a slow-decay head with positive-mean feature maps over a
 * long chunk; bf16 has the range of fp32 and no such limit.
 *
 * Every call only ENQUEUES work on `stream` (a hipStream_t; NULL = the default
 * stream); nothing is allocated, freed or synchronised, pointers are borrowed
 * until the enqueued work has run.  Return value: 0 on success, > 0 a
 * hipError_t, < 0 an argument error (LASP_E_*); lasp_last_error() then holds a
 * message for the calling thread.
 *
 * The entry points replace the Triton launches of the reference:
 *   lasp_chunk_fwd  <- lasp/lightning_attention.py:414-429 (_fwd_kernel, no state)
 *                      lasp/lasp_fuse.py:380-399 (_fwd_kernel with KV in/out)
 *                      lasp/lasp_fuse_parallel.py:852-942 (diag / kv_parallel /
 *                        kv_reduce / none_diag launches + the torch KV update)
 *   lasp_chunk_bwd  <- lasp/lightning_attention.py:459-502 (_bwd_intra_kernel,
 *                        _bwd_inter_kernel)
 *                      lasp/lasp_fuse.py:438-461 (_bwd_kernel with KV, DKV)
 *                      lasp/lasp_fuse_parallel.py:970-1068
 */
#ifndef LASP_HIP_H
#define LASP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LASP_ABI_VERSION 1

/* element types of q/k/v/o/do/dq/dk/dv */
#define LASP_DTYPE_F32 0
#define LASP_DTYPE_BF16 1
#define LASP_DTYPE_F16 2

/* argument errors (negative return values) */
#define LASP_E_NULL (-1)     /* a required pointer is NULL */
#define LASP_E_SHAPE (-2)    /* unsupported b/h/n/d/e */
#define LASP_E_DTYPE (-3)    /* unknown dtype code */
#define LASP_E_SEGMENT (-4)  /* seg_len invalid for this shape */
#define LASP_E_WORKSPACE (-5)/* workspace missing or too small */
#define LASP_E_ALIGN (-6)    /* a pointer is not aligned as the tensor contract asks */
#define LASP_E_DEVICE (-7)   /* q is not device memory of the calling thread's current device */
#define LASP_E_ALIAS (-8)    /* an outgoing state overlaps the incoming one where that is not supported */

/* Which kernel family a shape/dtype is served by (lasp_kernel_path). */
#define LASP_PATH_GENERIC 0 /* fp32-FMA kernels: any dtype, any n, d,e <= 128 */
#define LASP_PATH_MFMA 1    /* MFMA kernels, any n (a ragged tail is masked): bf16 / fp16 with d and e
                               multiples of 8 (rows narrower than 128 are read zero-extended), fp32 with
                               d = e = 128 */
#define LASP_PATH_MFMA_FUSED 2 /* short chunks of the 16-bit MFMA shapes called with seg_len = 0 (n <= 2048
                               and few enough segments that rebuilding a segment's incoming state from
                               the blocks before it -- at most 16 of them -- is cheaper than a pre-pass
                               and a scan): one launch
                               per direction; NO workspace is read or written (seg_states,
                               kv_seg_states and workspace may be NULL and are ignored) and the forward
                               leaves no segment states behind.  An explicit seg_len selects
                               LASP_PATH_MFMA instead. */

int lasp_abi_version(void);

/* Message of the last failing call made by this thread ("" if none). */
const char *lasp_last_error(void);

/*
 * Work decomposition.  A chunk of n tokens is cut into n_seg segments of
 * seg_len tokens (the last one may be shorter); segments of one (b, h) run in
 * parallel and are stitched by a decayed scan over their d x e states.
 * lasp_plan returns the default seg_len for a shape (pass it, or any other
 * positive multiple of 64, to the calls below); n_seg = ceil(n / seg_len) and
 * the byte size of ONE segment-state array are written through the pointers
 * (either may be NULL).  The array is opaque: the MFMA kernels keep every state
 * zero-extended to 128 x 128 floats, the generic ones as d x e.  Replaces the BLOCK/NUM_BLOCK choice of
 * lasp/lasp_fuse_parallel.py:1080-1085 and the `kv` buffer shape of :876.
 */
int lasp_plan(int b, int h, int64_t n, int d, int e, int dtype, int seg_len_or_0,
              int *seg_len, int *n_seg, size_t *state_bytes);

/* LASP_PATH_* for this shape under the default plan (seg_len = 0), or a negative LASP_E_* if it is
 * unsupported. */
int lasp_kernel_path(int b, int h, int64_t n, int d, int e, int dtype);

/*
 * Whether a call with this shape and seg_len (0 = default plan) may update its state in place:
 * kv_out == kv_in in lasp_chunk_fwd (backward = 0), dkv_out == dkv_in in lasp_chunk_bwd
 * (backward = 1).  Returns 1 or 0, or a negative LASP_E_*.  The pre-pass / scan / sweep kernels
 * read the incoming state and write the outgoing one from the same thread, in that order, so
 * there it is 1.  Where the sweeps themselves combine the states (LASP_PATH_MFMA_FUSED, and chunks
 * of at most 4 segments on the 16-bit kernels) several workgroups read the incoming state and
 * another one writes the outgoing state when it is done, with nothing ordering the two: it is 0
 * unless a single workgroup does both (forward with one segment).  The reference updates in place
 * (lasp/lasp_fuse.py:126-127,352-353); a caller that wants that where this returns 0 passes a
 * copy of the incoming state as kv_in / dkv_in.
 */
int lasp_inplace_ok(int b, int h, int64_t n, int d, int e, int dtype, int seg_len, int backward);

/*
 * Forward:  O = ((Q K^T) (.) M) V + diag(l^i) Q KV_in,   M_ij = l^(i-j) [j <= i]
 *           KV_out = l^n KV_in + sum_j l^(n-j) k_j^T v_j              (l = exp(-s_h))
 * kv_in  NULL = zero incoming state.  kv_out NULL = state not wanted.
 * kv_out may be the same buffer as kv_in (in-place update, as lasp/lasp_fuse.py:126-127) where
 * lasp_inplace_ok says so; the call returns LASP_E_ALIAS where it does not, and for buffers
 * that overlap without being the same.
 * seg_states: workspace of `state_bytes` (lasp_plan); on return it holds per-segment states (opaque:
 * the state entering each segment; each segment's own contribution with few segments, and for
 * heads whose decay wipes a state within one segment, which the scan leaves out; slots that nothing
 * reads are left unwritten), which
 * lasp_chunk_bwd accepts as `kv_seg_states` -- for the same inputs, seg_len and kv_in -- to skip
 * recomputing them.  It may be NULL when n_seg == 1 and kv_in == NULL and kv_out == NULL, and on
 * LASP_PATH_MFMA_FUSED.
 */
int lasp_chunk_fwd(const void *q, const void *k, const void *v, const float *s,
                   const float *kv_in, float *kv_out, void *o, float *seg_states,
                   int b, int h, int64_t n, int d, int e, int dtype, int seg_len,
                   void *stream);

/*
 * lasp_chunk_fwd without a workspace argument.  No counterpart in the reference: it is
 * for callers that cannot allocate device memory around the call (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  Same computation and
 * results as lasp_chunk_fwd; the segment states go to a scratch array of
 * LASP_STATIC_SCRATCH_BYTES that is part of the library's code object (each GPU the
 * library runs on holds its own copy until the process ends).  The call allocates and
 * frees nothing, on the host or the device.
 * Limit: b * h * n_seg states of 64 KiB (128 x 128 floats; d x e floats on the generic
 * path) must fit, i.e. at most 512 states on the MFMA path -- the headline shape
 * b=1 h=16 n=65536 with the default seg_len just fits; a larger call returns
 * LASP_E_WORKSPACE (a longer seg_len lowers n_seg).
 * The first call on a device looks the scratch's device address up (hipGetSymbolAddress, which
 * may also make the runtime load the library's code object on that device): make one call per
 * device before entering a region that must not do that, e.g. before starting a graph capture.
 * All calls on one GPU share that GPU's scratch: two calls whose work overlaps in time
 * on one GPU (different streams, or different threads) race on it.  The states are not
 * returned, so a backward of the same chunk recomputes them (kv_seg_states = NULL).
 */
#define LASP_STATIC_SCRATCH_BYTES (32u << 20)
int lasp_chunk_fwd_static(const void *q, const void *k, const void *v, const float *s,
                          const float *kv_in, float *kv_out, void *o,
                          int b, int h, int64_t n, int d, int e, int dtype, int seg_len,
                          void *stream);

/*
 * Backward (given dO and DKV_in = dL/dKV_out):
 *   dQ_i = sum_{j<=i} l^(i-j) (dO_i . v_j) k_j + l^i dO_i KV_in^T
 *   dK_j = sum_{i>=j} l^(i-j) (dO_i . v_j) q_i + l^(n-j) v_j DKV_in^T
 *   dV_j = sum_{i>=j} l^(i-j) (q_i . k_j) dO_i + l^(n-j) k_j DKV_in
 *   DKV_out = l^n DKV_in + sum_i l^i q_i^T dO_i                  (= dL/dKV_in)
 * kv_in / dkv_in NULL = zero.  dkv_out NULL = not wanted; may be the same buffer as dkv_in
 * (lasp/lasp_fuse.py:352-353) under the same rule as kv_out / kv_in in the forward.
 * kv_seg_states: the array lasp_chunk_fwd left in `seg_states` for the same
 * inputs, seg_len and kv_in, or NULL to recompute it (then `workspace` must
 * hold 2 * state_bytes, else 1 * state_bytes).
 */
int lasp_chunk_bwd(const void *q, const void *k, const void *v, const float *s,
                   const void *d_o, const float *kv_in, const float *dkv_in,
                   void *dq, void *dk, void *dv, float *dkv_out,
                   const float *kv_seg_states, float *workspace,
                   size_t workspace_bytes, int b, int h, int64_t n, int d, int e,
                   int dtype, int seg_len, void *stream);

/*
 * Measurement hook (no counterpart in the reference, which times nothing).
 * Between lasp_profile_begin and lasp_profile_end every kernel the library
 * launches is bracketed by two hipEvents on its launch stream (at most
 * max_launches of them; later launches go untimed).  lasp_profile_end waits for
 * the recorded events and returns, per kernel class, the summed duration in
 * milliseconds and the number of launches (arrays of LASP_KERNEL_CLASSES
 * entries; either may be NULL).  One profile at a time; launches may come from
 * any thread while it is open (each claims its slot atomically), begin and end
 * are called by one thread.
 */
#define LASP_KERNEL_CLASSES 6
#define LASP_KC_APPLY 0   /* la_apply: the block sweep producing O */
#define LASP_KC_STATE 1   /* la_seg_state: per-segment state pre-pass */
#define LASP_KC_SCAN 2    /* decayed scan over segment states */
#define LASP_KC_GENERIC 3 /* any kernel of the generic fp32-FMA family */
#define LASP_KC_BWD3 4    /* la_bwd3: dQ, dK and dV block sweeps in one launch */
#define LASP_KC_FUSED 5   /* la_fused_fwd / la_fused_bwd: a short chunk in one launch */
int lasp_profile_begin(int max_launches);
int lasp_profile_end(double *ms_per_class, int *launches_per_class);

/*
 * Second measurement hook (no counterpart in the reference): one launch of a kernel that only
 * streams -- n_rd read streams and n_wr write streams of bytes_each bytes (a multiple of 16384),
 * walked in 16 KiB pieces with 16-byte accesses and non-temporal stores, the way the sweeps walk
 * their token blocks, by `grid` workgroups of 256 threads.  Built mixes (reads:writes): 1:0, 2:0,
 * 4:0, 0:1, 1:1, 3:1 (the forward sweep's), 4:3 (the backward sweep's), 7:3 (what the backward
 * sweep really moves).  rd / wr are HOST arrays of device pointers, each 16-byte aligned.  The
 * caller times it (events on `stream`); the rate it reaches is the ceiling the sweeps are
 * compared with beside the published HBM peak.
 */
int lasp_stream_probe(const void *const *rd, int n_rd, void *const *wr, int n_wr, size_t bytes_each,
                      int grid, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LASP_HIP_H */
