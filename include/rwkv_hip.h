/*
 * rwkv_hip.h -- C ABI of librwkv_hip.so: the WKV recurrence family and depthwise_conv1d
 * for AMD MI355X (gfx950).
 *
 * Every entry point replaces one plain-pointer launcher of BlinkDL/RWKV-CUDA (the
 * `cuda_forward` / `cuda_backward` prototypes that each `*_op.cpp` shim declares) and keeps
 * that launcher's argument ORDER and meaning.  Differences, the same for all of them:
 *   - a leading `stream` (a hipStream_t passed as void*; NULL = the null stream); the
 *     reference launches on the legacy default stream;
 *   - an `int` status is returned (RWKV_OK or a negative RWKV_ERR_*); the reference only
 *     asserts.  Nothing is launched when a status other than RWKV_OK is returned;
 *   - backward passes that need device scratch take it from the caller as a trailing
 *     (workspace, workspace_bytes) pair whose size the matching *_workspace_bytes()
 *     function reports.  No entry point allocates or frees device memory, and none
 *     synchronises: work is enqueued on `stream` and the call returns.
 *   - T and the head size N = C / H are run-time values (the reference bakes -D_T_ and -D_N_ into its kernels).
 *     wkv5 (bf16 and fp32), wkv5a, wkv6 and wkv6_state take any N from 1 to 128 (C a multiple of H); 64 runs on the kernels
 *     written for it, every other size on kernels that keep one state row in the registers of one to four lanes.
 *     rwkv7 takes N = 64 only.
 *
 * bf16 tensors are passed as uint16_t* (raw bfloat16 bits).  All tensors are dense and
 * contiguous in the layouts named per function and must be 16-byte aligned (head sizes other than 64: any alignment
 * of the element type).
 * Pointers are device pointers on the current HIP device.
 */
#ifndef RWKV_HIP_H
#define RWKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t rwkv_bf16;

enum {
    RWKV_OK = 0,
    RWKV_ERR_SHAPE = -1,     /* a dimension is <= 0, an unsupported head size C / H, T not a multiple of the chunk, ... */
    RWKV_ERR_NULL = -2,      /* a required pointer is NULL */
    RWKV_ERR_ALIGN = -3,     /* a pointer is not 16-byte aligned */
    RWKV_ERR_WORKSPACE = -4, /* workspace missing or smaller than *_workspace_bytes() */
    RWKV_ERR_LAUNCH = -5     /* the HIP runtime refused a launch (see rwkv_last_hip_error) */
};

/* Text for a status code; never NULL. */
const char* rwkv_strerror(int status);
/* hipError_t value of the last failed launch in this thread (0 if none). */
int rwkv_last_hip_error(void);
/* ABI version of this header (bumped when a signature changes). */
int rwkv_abi_version(void);
/* The version this header describes: a client compiled against it (the torch shim, a cgo or ctypes binding) compares it
 * with rwkv_abi_version() of the library it has loaded and refuses a mismatch. */
#define RWKV_ABI_VERSION 4

/* A measuring aid (no counterpart in the reference): one pass over `bytes` of device memory as a read-only stream
 * (mode 0: src is read, 16 bytes of dst may be written), a write-only stream (mode 1: dst) or a copy (mode 2), so that a
 * benchmark can price kernels against what the memory system delivers for reads and for writes. */
int rwkv_hbm_probe(void* stream, int mode, const void* src, void* dst, size_t bytes);

/* Per-call options of the *_ex entry points below (no counterpart in the reference).  Every *_ex function is its
 * reference-signature sibling plus a trailing `flags` word; the sibling is the same call with flags = 0.  Nothing here is
 * process-wide: two threads may run different algorithms or pass subsets at the same time.
 *   RWKV_FLAG_SWEEPS : wkv5 / wkv6 / wkv6_state run the sequential fp32 recurrence kernels instead of the chunked
 *                      matrix-core kernels (second algorithm; the parity anchor of the chunked kernels).
 *   RWKV_PASS_*      : restrict a backward to a subset of its kernels so that a profiler can time one kernel per call
 *                      (no pass bit set = all of them).  Sequential kernels: GR (gr, gu, workspace), GV (gv), GK (gk, gw,
 *                      gs; reads the workspace GR left).  Chunked kernels: GR selects the first sweep (gr, gu, workspace),
 *                      GK the second (gk, gv, gw, gs); GV alone is empty.  Outputs of the passes left out are not written. */
#define RWKV_PASS_GR 1u
#define RWKV_PASS_GV 2u
#define RWKV_PASS_GK 4u
#define RWKV_PASS_ALL 7u
#define RWKV_FLAG_SWEEPS 0x100u
/*   RWKV_FLAG_WHOLE  : rwkv_wkv6f_forward / rwkv_wkv6f_backward_saved keep one workgroup per (batch, head) also where
 *                      B H is below the number of CUs (by default such shapes run as several blocks per sequence joined
 *                      by a scan).  Forward and backward of one step must agree on it. */
#define RWKV_FLAG_WHOLE 0x200u

/* ---------------------------------------------------------------------------------------
 * RWKV-4 wkv, fp32.  Replaces cuda_forward / cuda_backward of wkv/cuda/wkv_op.cpp:3-4
 * (kernels: wkv/cuda/wkv_cuda_v2.cu:4-130).
 *   w[C]  = -exp(w_raw) (the wrapper's pre-transform, wkv/run.py:95), u[C], k,v,y,gy,gk,gv[B,T,C].
 *   gw,gu[B,C] are per-batch partials that the kernel ADDS into (caller zero-fills, as
 *   wkv/run.py:110-111 does); gw already carries the factor w of the w_raw chain rule.
 *   Where the reference keeps the backward's per-step intermediates in per-thread arrays of 4096 floats, here they stay
 *   in registers up to T = 32768 and go to gk, gv and the workspace (B*T*C floats) beyond, so T is not limited; the
 *   workspace is asked for at every T.
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv4_forward(void* stream, int B, int T, int C,
                      const float* w, const float* u, const float* k, const float* v, float* y);
size_t rwkv_wkv4_backward_workspace_bytes(int B, int T, int C);
int rwkv_wkv4_backward(void* stream, int B, int T, int C,
                       const float* w, const float* u, const float* k, const float* v, const float* gy,
                       float* gw, float* gu, float* gk, float* gv,
                       void* workspace, size_t workspace_bytes);

/* rwkv_wkv4_backward without a workspace argument and without any allocation.  It has no counterpart in the reference;
 * it is for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  Only the kernels for T > 32768 (or B > 65535) need scratch memory, B*T*C floats: it lives in
 * a file-scope device array of the library, rwkv_wkv4_backward_noalloc_max_elems() floats (8 MiB) that every GPU the
 * library runs on holds until the process ends, and for those shapes B*T*C beyond that returns RWKV_ERR_WORKSPACE.
 * Shorter sequences use no scratch and have no size limit.  All calls on one GPU share the one array: calls that use it
 * and overlap in time on the same GPU (two streams, two threads) race; serialise them.  Results are those of
 * rwkv_wkv4_backward. */
size_t rwkv_wkv4_backward_noalloc_max_elems(void);
int rwkv_wkv4_backward_noalloc(void* stream, int B, int T, int C,
                               const float* w, const float* u, const float* k, const float* v, const float* gy,
                               float* gw, float* gu, float* gk, float* gv);

/* The whole of WKV.forward / WKV.backward (wkv/run.py:89-117) behind two calls: w_raw[C] is the raw parameter (the kernels
 * apply w = -exp(w_raw), :95), and gw, gu [C] come out summed over the batch (:115-116; no zero-fill by the caller).  The
 * backward launches the sweep kernel and one small reduction kernel; the order of every sum is fixed.  Workspace: the
 * B*T*C floats of rwkv_wkv4_backward plus 2*B*C floats of per-batch partials. */
int rwkv_wkv4raw_forward(void* stream, int B, int T, int C,
                         const float* w_raw, const float* u, const float* k, const float* v, float* y);
size_t rwkv_wkv4raw_backward_workspace_bytes(int B, int T, int C);
int rwkv_wkv4raw_backward(void* stream, int B, int T, int C,
                          const float* w_raw, const float* u, const float* k, const float* v, const float* gy,
                          float* gw, float* gu, float* gk, float* gv,
                          void* workspace, size_t workspace_bytes);

/* ---------------------------------------------------------------------------------------
 * depthwise_conv1d ("TimeX"), fp32.  Replaces cuda_forward / cuda_backward of
 * depthwise_conv1d/cuda/timex_op.cpp:3-4 (kernels: timex_cuda_v3.cu:7-150).
 *   w[C,T], k,x,gwk,gk[B,C,T];  x[b,c,t] = eps + sum_{u<=t} w[c,T-1-(t-u)] k[b,c,u].
 *   gw[B,C,T] is per batch (the wrapper sums over B, depthwise_conv1d/run.py:102).
 *   T must be a multiple of 4 (same as the reference); B is unrestricted.
 *   With T % 32 == 0, T <= 1024 and B >= 8 the sums run on the matrix cores with every fp32 operand carried as two fp16
 *   terms (22 mantissa bits, scaled by a power of two per 32 batch rows): errors against fp64 are those of an fp32 loop
 *   (1e-7 of the outputs' scale), but a product is not the bit pattern of the fp32 product.
 * ------------------------------------------------------------------------------------- */
int rwkv_timex_forward(void* stream, const float* w, const float* k, float* x, float eps, int B, int C, int T);
int rwkv_timex_backward(void* stream, const float* w, const float* k, const float* gwk,
                        float* gw, float* gk, int B, int C, int T);
/* The same backward with the wrapper's sum over the batch (depthwise_conv1d/run.py:102) done inside:
 * gw_sum[C,T] = sum_b gw[b], gk as above.  Needs T % 32 == 0 and T <= 1024 (RWKV_ERR_SHAPE otherwise:
 * call rwkv_timex_backward and sum).  The order of every fp32 sum is fixed, so results repeat bit for bit. */
int rwkv_timex_backward_sum(void* stream, const float* w, const float* k, const float* gwk,
                            float* gw_sum, float* gk, int B, int C, int T);

/* ---------------------------------------------------------------------------------------
 * RWKV-5 wkv, bf16 I/O.  Replaces cuda_forward / cuda_backward of
 * wkv5_bf16/cuda/wkv5_op.cpp:5-6 (kernels: wkv5_cuda_v1b.cu:6-191).
 *   r,k,v,y,gy,gr,gk,gv[B,T,C] bf16; eew = exp(-exp(w_raw)) and ew = -exp(w_raw), fp32 [H,N]
 *   (wkv5_bf16/run.py:63-64); u[H,N] bf16; gw,gu[B,C] bf16 per-batch partials (fully written).
 *   Backward workspace (wkv5, wkv6, wkv6_state alike): B*T*C floats (r * dr' between the two sweeps) followed by one
 *   64x64 fp32 forward state per (b,h) and 128 tokens; private to the library, no initialisation needed.  wkv5 with heads
 *   of 128 channels asks for more (fp32 terms of gr, gk, gv, gw, gu): take the size from the function below.
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv5_forward(void* stream, int B, int T, int C, int H,
                      const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                      const float* eew, const rwkv_bf16* u, rwkv_bf16* y);
int rwkv_wkv5_forward_ex(void* stream, int B, int T, int C, int H,
                      const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                      const float* eew, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags);
/* The forward with a workspace.  It has no counterpart in the reference (whose forward takes none): heads of 128 channels
 * run on the matrix-core kernels as four heads of 64 whose fp32 terms are added afterwards, and those terms need
 * rwkv_wkv5_forward_workspace_bytes() of scratch (B*T*C floats; 0 for every other head size, which then needs no
 * workspace and runs exactly as rwkv_wkv5_forward_ex).  Without it heads of 128 take the one-row-per-lane kernels. */
size_t rwkv_wkv5_forward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv5_forward_ws(void* stream, int B, int T, int C, int H,
                         const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const float* eew, const rwkv_bf16* u, rwkv_bf16* y,
                         void* workspace, size_t workspace_bytes, unsigned flags);
size_t rwkv_wkv5_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv5_backward(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const float* eew, const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes);
int rwkv_wkv5_backward_ex(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const float* eew, const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes, unsigned flags);

/* WKV_5.forward / backward (wkv5_bf16/run.py:44-88) with the wrapper's steps folded in.  w_raw[H,N] is the raw bf16
 * parameter; the forward writes decay[2*C] fp32 = [exp(-exp(w_raw)) | -exp(w_raw)] (:63-64), which the caller keeps for the
 * backward; gw, gu [H,N] bf16 come out summed over the batch exactly as torch.sum over the bf16 per-batch partials gives
 * them (:86-87).  `flags` as for the *_ex entry points. */
int rwkv_wkv5raw_forward(void* stream, int B, int T, int C, int H,
                         const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay, unsigned flags);
int rwkv_wkv5raw_forward_ws(void* stream, int B, int T, int C, int H,
                            const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                            const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay,
                            void* workspace, size_t workspace_bytes, unsigned flags);   /* see rwkv_wkv5_forward_ws */
size_t rwkv_wkv5raw_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv5raw_backward(void* stream, int B, int T, int C, int H,
                          const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                          const float* decay, const rwkv_bf16* u, const rwkv_bf16* gy,
                          rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                          void* workspace, size_t workspace_bytes, unsigned flags);

/* ---------------------------------------------------------------------------------------
 * RWKV-5 wkv, fp32 I/O.  Replaces cuda_forward / cuda_backward of wkv5/cuda/wkv5_op.cpp:3-4
 * (kernels: wkv5_cuda_v1e.cu and its siblings, selected by CUDA_KERNEL_VERSION in wkv5/run.py:15).
 *   Same arguments as the bf16 op with every tensor fp32; gw,gu[B,C] fp32 per-batch partials
 *   (wkv5/run.py:497-501 sums them over the batch).  Head size 64 only: the reference compiles N
 *   in (wkv5/run.py:467) and benchmarks N = 64.
 *   Runs the sequential fp32 sweeps; the decay gradient comes from the reference's own second
 *   recurrence (dS/dw carried forward in time), so the backward needs no workspace.
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv5f32_forward(void* stream, int B, int T, int C, int H,
                         const float* r, const float* k, const float* v,
                         const float* eew, const float* u, float* y);
int rwkv_wkv5f32_backward(void* stream, int B, int T, int C, int H,
                          const float* r, const float* k, const float* v,
                          const float* eew, const float* ew, const float* u, const float* gy,
                          float* gr, float* gk, float* gv, float* gw, float* gu);
int rwkv_wkv5f32_backward_ex(void* stream, int B, int T, int C, int H,
                          const float* r, const float* k, const float* v,
                          const float* eew, const float* ew, const float* u, const float* gy,
                          float* gr, float* gk, float* gv, float* gw, float* gu, unsigned flags);

/* ---------------------------------------------------------------------------------------
 * wkv5a: RWKV-5 wkv with two-sided decay and bonus, fp32.  Replaces cuda_forward / cuda_backward of
 * wkv5a/cuda/wkv5a_op.cpp:6-7 (kernels: wkv5a_cuda_v1a2.cu:7-222; DTYPE = float, :5).
 *   State element [i = value channel][j = key channel] decays by eew1[j] * eew2[i] and the current
 *   token's bonus is u1[j] + u2[i].  eewX = exp(-exp(wX_raw)), ewX = -exp(wX_raw), fp32 [H,N]
 *   (wkv5a/run.py:123-126); gw1,gu1,gw2,gu2[B,C] fp32 per-batch partials w.r.t. the raw parameters
 *   (summed over the batch by the wrapper, wkv5a/run.py:150-153).  Head size 64.  No workspace.
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv5a_forward(void* stream, int B, int T, int C, int H,
                       const float* r, const float* k, const float* v,
                       const float* eew1, const float* u1, const float* eew2, const float* u2, float* y);
int rwkv_wkv5a_backward(void* stream, int B, int T, int C, int H,
                        const float* r, const float* k, const float* v,
                        const float* eew1, const float* ew1, const float* u1,
                        const float* eew2, const float* ew2, const float* u2, const float* gy,
                        float* gr, float* gk, float* gv, float* gw1, float* gu1, float* gw2, float* gu2);
int rwkv_wkv5a_backward_ex(void* stream, int B, int T, int C, int H,
                        const float* r, const float* k, const float* v,
                        const float* eew1, const float* ew1, const float* u1,
                        const float* eew2, const float* ew2, const float* u2, const float* gy,
                        float* gr, float* gk, float* gv, float* gw1, float* gu1, float* gw2, float* gu2, unsigned flags);

/* ---------------------------------------------------------------------------------------
 * RWKV-6 wkv, bf16 I/O, per-token decay.  Replaces cuda_forward / cuda_backward of
 * wkv6/cuda/wkv6_op.cpp:5-6 (kernels: wkv6_cuda_v1.cu:6-223).
 *   w = ew = -exp(w_raw), fp32 [B,T,C] (wkv6/run.py:147); the kernel applies exp(ew).
 *   gw[B,T,C] bf16 is the gradient w.r.t. w_raw and is fully written (rows 0 and T-1 are
 *   exact zeros, which is what the reference leaves in its pre-zeroed buffer); gu[B,C].
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv6_forward(void* stream, int B, int T, int C, int H,
                      const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                      const float* ew, const rwkv_bf16* u, rwkv_bf16* y);
int rwkv_wkv6_forward_ex(void* stream, int B, int T, int C, int H,
                      const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                      const float* ew, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags);
size_t rwkv_wkv6_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv6_backward(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes);
int rwkv_wkv6_backward_ex(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const float* ew, const rwkv_bf16* u, const rwkv_bf16* gy,
                       rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                       void* workspace, size_t workspace_bytes, unsigned flags);

/* RWKV-6 wkv without state, taking the RAW bf16 decay parameter w[B,T,C] (the kernels apply exp(-exp(w)) and
 * return gw w.r.t. w): the wrapper-side pre-transform ew = -exp(w.float()) of wkv6/run.py:147 folded into the
 * kernels, which removes an fp32 [B,T,C] temporary and three elementwise passes.  No counterpart in the reference's
 * C++ shim; the Python class WKV_6 keeps its reference signature and calls these. */
int rwkv_wkv6raw_forward(void* stream, int B, int T, int C, int H,
                         const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const rwkv_bf16* w, const rwkv_bf16* u, rwkv_bf16* y);
int rwkv_wkv6raw_forward_ex(void* stream, int B, int T, int C, int H,
                         const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                         const rwkv_bf16* w, const rwkv_bf16* u, rwkv_bf16* y, unsigned flags);
int rwkv_wkv6raw_backward(void* stream, int B, int T, int C, int H,
                          const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                          const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* gy,
                          rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                          void* workspace, size_t workspace_bytes);
int rwkv_wkv6raw_backward_ex(void* stream, int B, int T, int C, int H,
                          const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                          const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* gy,
                          rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                          void* workspace, size_t workspace_bytes, unsigned flags);

/* The backward of WKV_6 (s = gs = NULL) and WKV_6STATE with the wrapper's torch.sum(gu, 0) (wkv6/run.py:169,
 * wkv6_state/run.py:123) folded in: raw bf16 w, gu[H,N] summed over the batch as torch.sum over the bf16 per-batch
 * partials gives it.  The forward is rwkv_wkv6raw_forward / rwkv_wkv6state_forward.  `flags` as for the *_ex entry points. */
size_t rwkv_wkv6f_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv6f_backward(void* stream, int B, int T, int C, int H,
                        const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                        const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy,
                        rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                        rwkv_bf16* gs, void* workspace, size_t workspace_bytes, unsigned flags);

/* WKV_6 (s = gs = NULL) and WKV_6STATE with states handed from the forward to the backward.  The forward also writes,
 * into `saved` (rwkv_wkv6f_saved_bytes; [B*H][ceil(T/64)] states of 64 x 64 values in 12 KB each: fp32 rounded to 24
 * bits, in an order private to the two kernels), the state entering every 64th token; the backward reads them and produces every gradient in ONE reverse sweep instead of two sweeps and an fp32 [B,T,C] hand-over.  The
 * reference's wkv6 operators keep nothing between their two calls; the precedents are its rwkv7 forward, which keeps `s`
 * and `sa` for its backward (rwkv7_statepassing_clampw.cu:67-73), and wkv5_bf16/cuda/wkv5_cuda_v3.cu:12-30 (chunk states).
 * Results are those of the pair above to the rounding of the outputs.  With another head size than 64, or with
 * RWKV_FLAG_SWEEPS / RWKV_PASS_*, rwkv_wkv6f_saved_bytes is 0 for sizes the kernels do not take, `saved` may be NULL and
 * both calls run the kernels above.  The workspace also serves the two-sweep kernels, which redo any (batch, head) whose
 * decay over 16 tokens exceeds e^-60. */
size_t rwkv_wkv6f_saved_bytes(int B, int T, int C, int H);
int rwkv_wkv6f_forward(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, rwkv_bf16* y,
                       void* saved, size_t saved_bytes, unsigned flags);
size_t rwkv_wkv6f_backward_saved_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv6f_backward_saved(void* stream, int B, int T, int C, int H,
                              const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                              const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy,
                              rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                              rwkv_bf16* gs, const void* saved, size_t saved_bytes,
                              void* workspace, size_t workspace_bytes, unsigned flags);

/* The same pair for wkv5 at head size 64 (no counterpart in the reference; what WKV_5 of wkv5_bf16/run.py:44-88 does in
 * two calls, its wrapper's decay transforms and sums included): raw bf16 w[H,N] in, y out, `decay` = [eew | ew] (2 C
 * floats) left by the forward for the backward, gw, gu [H,N] summed over time and batch out.  The decay of a channel
 * stands in for every token's decay in the kernels of rwkv_wkv6f_*, and its gradient is added up over the tokens inside
 * the kernel.  Other head sizes, RWKV_FLAG_SWEEPS / RWKV_PASS_* or saved = NULL: rwkv_wkv5raw_forward / _backward. */
size_t rwkv_wkv5s_saved_bytes(int B, int T, int C, int H);
int rwkv_wkv5s_forward(void* stream, int B, int T, int C, int H,
                       const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                       const rwkv_bf16* w_raw, const rwkv_bf16* u, rwkv_bf16* y, float* decay,
                       void* saved, size_t saved_bytes, unsigned flags);
size_t rwkv_wkv5s_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv5s_backward(void* stream, int B, int T, int C, int H,
                        const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                        const rwkv_bf16* w_raw, const float* decay, const rwkv_bf16* u, const rwkv_bf16* gy,
                        rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                        const void* saved, size_t saved_bytes, void* workspace, size_t workspace_bytes, unsigned flags);

/* ---------------------------------------------------------------------------------------
 * RWKV-6 wkv with initial state.  Replaces cuda_forward / cuda_backward of
 * wkv6_state/cuda/wkv6state_op.cpp:5-6 (kernels: wkv6state_cuda_v1a.cu:6-308).
 *   w[B,T,C] is the RAW bf16 decay parameter; the kernel applies exp(-exp(w)).
 *   s,gs[B,H,N,N] bf16, indexed [value channel][key channel]; every output is fully written.
 * ------------------------------------------------------------------------------------- */
int rwkv_wkv6state_forward(void* stream, int B, int T, int C, int H,
                           const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                           const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, rwkv_bf16* y);
int rwkv_wkv6state_forward_ex(void* stream, int B, int T, int C, int H,
                           const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                           const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, rwkv_bf16* y, unsigned flags);
size_t rwkv_wkv6state_backward_workspace_bytes(int B, int T, int C, int H);
int rwkv_wkv6state_backward(void* stream, int B, int T, int C, int H,
                            const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                            const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy,
                            rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                            rwkv_bf16* gs, void* workspace, size_t workspace_bytes);
int rwkv_wkv6state_backward_ex(void* stream, int B, int T, int C, int H,
                            const rwkv_bf16* r, const rwkv_bf16* k, const rwkv_bf16* v,
                            const rwkv_bf16* w, const rwkv_bf16* u, const rwkv_bf16* s, const rwkv_bf16* gy,
                            rwkv_bf16* gr, rwkv_bf16* gk, rwkv_bf16* gv, rwkv_bf16* gw, rwkv_bf16* gu,
                            rwkv_bf16* gs, void* workspace, size_t workspace_bytes, unsigned flags);

/* ---------------------------------------------------------------------------------------
 * RWKV-7 "clamp-w" with state passing, bf16 I/O, fp32 states.  Replaces cuda_forward /
 * cuda_backward of rwkv7_fast_fused/cuda/rwkv7_statepassing_clampw.cpp:10,17
 * (kernels: rwkv7_statepassing_clampw.cu:20-193).
 *   r,w,k,v,a,b,y,dy,dr,dw,dk,dv,da,db [B,T,H,N] bf16 (w raw; decay = exp(-e^-0.5 * sigmoid(w)));
 *   s0,sT,dsT,ds0 [B,H,N,N] fp32 indexed [value][key];
 *   s  [B,H,T/16,N,N] fp32 : state checkpoints written by forward, read by backward;
 *   sa [B,T,H,N]      fp32 : S_t a_t written by forward, read by backward.
 *   T must be a multiple of RWKV7_CHUNK_LEN (16), as rwkv7_statepassing_clampw.cu:191 asserts.
 *   The layout inside `s` is private to this library (forward and backward must both come
 *   from it).
 * ------------------------------------------------------------------------------------- */
#define RWKV7_CHUNK_LEN 16
int rwkv7_statepassing_forward(void* stream, int B, int T, int H,
                               const float* s0, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
                               const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                               rwkv_bf16* y, float* sT, float* s, float* sa);
int rwkv7_statepassing_backward(void* stream, int B, int T, int H,
                                const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v,
                                const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy, const float* dsT,
                                const float* s, const float* sa, float* ds0,
                                rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                                rwkv_bf16* da, rwkv_bf16* db);

/* The state-passing op with the per-call flags word (RWKV_FLAG_SWEEPS: the step-by-step recurrence kernels instead of
 * the chunked matrix-core kernels).  PAIRING RULE: the two families lay `s` out differently (the chunked kernels store
 * the state entering each chunk, the step kernels, like the reference, the state leaving it) and `s` carries no tag, so a
 * backward must be given the flags of the forward that wrote its `s` and `sa`.  The entry points without a flags word
 * (rwkv7_*_forward / _backward, and through them the torch shim) are the chunked family: a forward_ex with
 * RWKV_FLAG_SWEEPS followed by one of those backwards is undefined -- wrong gradients, no error.  The Python wrapper
 * keeps the flags of the forward on the autograd context for this reason.  Here s0 and sT (forward), dsT and ds0 (backward) may be NULL: a missing s0 / dsT is zero, a missing
 * sT / ds0 is not written.  No counterpart in the reference. */
int rwkv7_statepassing_forward_ex(void* stream, int B, int T, int H,
                                  const float* s0, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
                                  const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                                  rwkv_bf16* y, float* sT, float* s, float* sa, unsigned flags);
int rwkv7_statepassing_backward_ex(void* stream, int B, int T, int H,
                                   const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v,
                                   const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy, const float* dsT,
                                   const float* s, const float* sa, float* ds0,
                                   rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                                   rwkv_bf16* da, rwkv_bf16* db, unsigned flags);

/* The two siblings of the state-passing op, served by the same kernels:
 *   rwkv7_state_*  : initial state s0 and its gradient ds0, no final state.  Replaces cuda_forward /
 *                    cuda_backward of rwkv7_fast_fused/cuda/rwkv7_state_clampw.cpp:10,17.
 *   rwkv7_forward / rwkv7_backward : zero initial state, no state outputs.  Replaces cuda_forward /
 *                    cuda_backward of rwkv7_fast_fused/cuda/rwkv7_clampw.cpp:10,17.
 * Argument order is the reference's after the leading stream.  These are the bf16 mode; the *_f32 entry points below
 * are the reference's -D_FP32_ build. */
int rwkv7_state_forward(void* stream, int B, int T, int H,
                        const float* s0, const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k,
                        const rwkv_bf16* v, const rwkv_bf16* a, const rwkv_bf16* b,
                        rwkv_bf16* y, float* s, float* sa);
int rwkv7_state_backward(void* stream, int B, int T, int H,
                         const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v,
                         const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy,
                         const float* s, const float* sa, float* ds0,
                         rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                         rwkv_bf16* da, rwkv_bf16* db);
int rwkv7_forward(void* stream, int B, int T, int H,
                  const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v,
                  const rwkv_bf16* a, const rwkv_bf16* b, rwkv_bf16* y, float* s, float* sa);
int rwkv7_backward(void* stream, int B, int T, int H,
                   const rwkv_bf16* r, const rwkv_bf16* w, const rwkv_bf16* k, const rwkv_bf16* v,
                   const rwkv_bf16* a, const rwkv_bf16* b, const rwkv_bf16* dy,
                   const float* s, const float* sa,
                   rwkv_bf16* dr, rwkv_bf16* dw, rwkv_bf16* dk, rwkv_bf16* dv,
                   rwkv_bf16* da, rwkv_bf16* db);

/* fp32 I/O for the three rwkv7 ops: what the reference builds from the same sources with -D_FP32_, where `bf` is float
 * (rwkv7_clampw.cu:3-7, rwkv7_cuda_benchmark.py:102-126, and the same lines of the _state and _state_passing siblings).
 * Same arguments as the bf16 entry points with every bf16 tensor fp32; same kernels and fp32 arithmetic. */
int rwkv7_statepassing_forward_f32(void* stream, int B, int T, int H,
                                   const float* s0, const float* r, const float* w, const float* k,
                                   const float* v, const float* a, const float* b,
                                   float* y, float* sT, float* s, float* sa);
int rwkv7_statepassing_backward_f32(void* stream, int B, int T, int H,
                                    const float* r, const float* w, const float* k, const float* v,
                                    const float* a, const float* b, const float* dy, const float* dsT,
                                    const float* s, const float* sa, float* ds0,
                                    float* dr, float* dw, float* dk, float* dv, float* da, float* db);
int rwkv7_state_forward_f32(void* stream, int B, int T, int H,
                            const float* s0, const float* r, const float* w, const float* k,
                            const float* v, const float* a, const float* b, float* y, float* s, float* sa);
int rwkv7_state_backward_f32(void* stream, int B, int T, int H,
                             const float* r, const float* w, const float* k, const float* v,
                             const float* a, const float* b, const float* dy,
                             const float* s, const float* sa, float* ds0,
                             float* dr, float* dw, float* dk, float* dv, float* da, float* db);
int rwkv7_forward_f32(void* stream, int B, int T, int H,
                      const float* r, const float* w, const float* k, const float* v,
                      const float* a, const float* b, float* y, float* s, float* sa);
int rwkv7_backward_f32(void* stream, int B, int T, int H,
                       const float* r, const float* w, const float* k, const float* v,
                       const float* a, const float* b, const float* dy,
                       const float* s, const float* sa,
                       float* dr, float* dw, float* dk, float* dv, float* da, float* db);

#ifdef __cplusplus
}
#endif
#endif /* RWKV_HIP_H */
