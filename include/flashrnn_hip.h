/* C ABI of libflashrnn_hip.so: the MI355X (gfx950) recurrent hot path of FlashRNN.
 *
 * Each entry point replaces one method of the reference's per-configuration pybind objects
 *   FlashRNNFuncFused {forward, backward}   flashrnn/flashrnn/fused/flashrnn.cc:55-346
 *   FlashRNNFunc      {forward, backward}   flashrnn/flashrnn/alternating/flashrnn.cc:39-313
 * and, below them, ForwardPass::Run / BackwardPass::Run
 *   flashrnn/flashrnn/fused/flashrnn.h:118-150, flashrnn/flashrnn/alternating/flashrnn.h:48-369.
 *
 * Differences in contract (all on purpose):
 *  - one library for every (function, dtype, head dim): the configuration is passed at run
 *    time, nothing is JIT-compiled (reference: one nvcc build per config, cuda_init.py:95-168);
 *  - tensors are read and written in the PUBLIC layouts of flashrnn() (flashrnn.py:165-173):
 *      Wx [B,T,G_w,N,D]   R [G_r,N,D,D] (out unit, previous unit)   b [G_t,N,D]
 *      s0 [S,B,N,D]       states [S,B,T,N,D]       dstates [S,B,T,N,D]
 *    so the caller makes no permuted copies (reference: flashrnn.py:1130-1133, :1053);
 *  - the batch is padded to the MFMA tile inside the kernels; B is the true batch size
 *    (reference pads in Python, flashrnn.py:699-717);
 *  - the library allocates nothing: outputs, the gate cache and a workspace are the caller's,
 *    sized by the *_bytes queries; every call runs on the stream it is given and is
 *    asynchronous; there are no device-wide synchronisations
 *    (reference: cudaDeviceSynchronize in flashrnn_fused_backward.cu:1001);
 *  - dR and db are returned in fp32 whatever the storage type (reference: storage type).
 *
 * All pointers are device pointers, 16-byte aligned, tensors contiguous.  Element type is
 * bf16 (FRNN_BF16), fp16 (FRNN_F16) or fp32 (FRNN_F32) for Wx, R, b, s0, states, dstates, dWx,
 * ds0.  Whatever the storage type, MFMA accumulation and all gate math are fp32 (the reference
 * accumulates fp16 in fp16 and computes the gates in the storage type).
 *
 * Return value: 0 ok; negative = argument error found on the host before any launch
 * (FRNN_E_*; text in frnn_last_error()); positive = hipError_t of a failed launch.
 */
#ifndef FLASHRNN_HIP_H
#define FLASHRNN_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* function ids: gate/state counts as in flashrnn.py:49-71 */
enum { FRNN_LSTM = 0, FRNN_SLSTM = 1, FRNN_GRU = 2, FRNN_ELMAN = 3 };
enum { FRNN_BF16 = 0, FRNN_F32 = 1, FRNN_F16 = 2 };  /* DTYPE_DICT, flashrnn.py:73-78 */

enum {
  FRNN_OK = 0,
  FRNN_E_ARG = -1,         /* unknown function / dtype, non-positive size */
  FRNN_E_UNSUPPORTED = -2, /* no kernel for this (function, dtype, D); use the other backend */
  FRNN_E_NULL = -3,        /* a required pointer is null */
  FRNN_E_ALIGN = -4,       /* a pointer is not 16-byte aligned */
  FRNN_E_WORKSPACE = -5,   /* workspace smaller than frnn_*_workspace_bytes() */
  FRNN_E_DEVICE = -6,      /* current device is not usable (query failed, too few CUs) */
  FRNN_E_TOO_LARGE = -7    /* fused backend: a tensor of this call reaches 2 GiB (32-bit offsets inside the kernels); run the
                            * batch as ranges of at most frnn_fused_max_batch() rows, see frnn_options.batch_stride */
};

/* Thread-local text of the last error returned on this thread ("" if none). */
const char* frnn_last_error(void);
const char* frnn_version(void);

/* Optional per-launch timing with HIP events on the caller's stream (off by default; for
 * benchmarks: one thread, one stream).  No counterpart in the reference, which prints occupancy
 * and register use at build time instead (cuda_init.py:144-147).  frnn_profile_enable(1) starts
 * recording; each entry is one kernel launch (or the per-step launch loop of the alternating
 * backend); frnn_profile_ms(i) waits for entry i and returns its duration in milliseconds. */
void frnn_profile_enable(int on);
void frnn_profile_reset(void);
int frnn_profile_count(void);
const char* frnn_profile_name(int i);
float frnn_profile_ms(int i);

/* (G_r, G_w, G_t, S) of a function and the number of values per element the gate cache
 * holds; 0 ok / FRNN_E_ARG.  Mirrors rnn_function_registry, flashrnn.py:49-71. */
int frnn_function_dims(int function, int* G_r, int* G_w, int* G_t, int* S, int* cache_vals);

/* ---- fused backend ("hip_fused"): replaces FlashRNNFuncFused, fused/flashrnn.cc:55-346 ---- */

/* 0 if a fused kernel exists for (function, dtype, D) and B,N fit the device, else FRNN_E_*.
 * Replaces the reference's "does a tiling exist" search (flashrnn.py:429-589). */
int frnn_fused_supported(int function, int dtype, int B, int N, int D);

/* The launch plan: waves per workgroup, 16-unit tiles per wave, workgroups per head and the
 * number of workgroups that do work (= compute units used; heads that run as one workgroup of
 * up to 4 waves may share a compute unit three at a time).  backward = 0/1. */
int frnn_fused_plan(int function, int dtype, int B, int N, int D, int backward,
                    int* waves, int* tiles_per_wave, int* wgs_per_head, int* active_wgs);

/* Bytes of the private gate cache written by a training forward and read by backward
 * (reference: gate_cache_r / gate_cache_i, fused/flashrnn.cc:97-112). */
size_t frnn_fused_cache_bytes(int function, int dtype, int B, int T, int N, int D);

/* Bytes of workspace for forward (backward = 0) or backward (backward = 1).  The first
 * 4 bytes of the workspace hold a status word after the call: 0 ok, 1 = a bounded wait
 * between workgroups ran out (the outputs are then filled with NaN from that step on). */
size_t frnn_fused_workspace_bytes(int function, int dtype, int B, int T, int N, int D, int backward);

/* Concurrency: when a head spans several workgroups (frnn_fused_plan: wgs_per_head > 1) they wait for
 * each other inside the kernel and must all be resident.  Launches of such kernels on different streams of
 * one device are ordered behind each other by the library (an event wait on the device, nothing blocks on
 * the host; the reference's cooperative launch gives the same guarantee, fused/flashrnn_fused_forward.cu:
 * 893-911); FRNN_COOPERATIVE=1 in the environment launches them as cooperative kernels instead (about 15 us
 * more per launch).  Kernels of other processes are not seen: every wait is bounded, and a wait that runs out
 * is reported in the status word instead of hanging.
 * The workgroups of a head exchange h (forward) and partial sums (backward) through tagged words in the
 * workspace.  A launch places them on one XCD and the kernels check that at their start; the exchange stores
 * then stay in that XCD's L2.  Where the check fails, or with FRNN_AGENT_STORES=1, they are written through to
 * memory (slower, same results). */

/* Forward over the whole sequence.  Replaces FlashRNNFuncFused::forward (fused/flashrnn.cc:68-144)
 * + ForwardPass::Run (fused/flashrnn_fused_forward.cu:772-975).
 *   training != 0: also fills `cache` (frnn_fused_cache_bytes); else cache may be null.
 *   states [S,B,T,N,D] receives s_1..s_T (s0 is NOT copied in front, unlike the reference's
 *   [S,T+1,B,N,D] buffer). */
int frnn_fused_forward(int function, int dtype, int training, int B, int T, int N, int D,
                       const void* Wx, const void* R, const void* b, const void* s0,
                       void* states, void* cache, void* workspace, size_t workspace_bytes,
                       void* stream);

/* Backward.  Replaces FlashRNNFuncFused::backward (fused/flashrnn.cc:146-246) +
 * BackwardPass::Run (fused/flashrnn_fused_backward.cu:768-1086) including its post-loop
 * dR GEMM (:1049-1055) and bias reduction (:626-665).
 *   dstates [S,B,T,N,D]: cotangent of every output state.
 *   outputs: dWx [B,T,G_w,N,D], ds0 [S,B,N,D] (storage type); dR [G_r,N,D,D], db [G_t,N,D] (fp32). */
int frnn_fused_backward(int function, int dtype, int B, int T, int N, int D,
                        const void* R, const void* b, const void* s0, const void* states,
                        const void* cache, const void* dstates,
                        void* dWx, void* ds0, float* dR, float* db,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ---- alternating backend ("hip"): replaces FlashRNNFunc, alternating/flashrnn.cc:39-313 ---- */

int frnn_alt_supported(int function, int dtype, int B, int N, int D);
size_t frnn_alt_cache_bytes(int function, int dtype, int B, int T, int N, int D);
size_t frnn_alt_workspace_bytes(int function, int dtype, int B, int T, int N, int D, int backward);

/* One kernel launch per time step: R h_{t-1} of a 16-unit x 16-row tile on MFMA, then its gate
 * math (the reference launches a cuBLAS GEMM and a pointwise kernel per step).
 * Replaces ForwardPass::Run / IterateInternal, alternating/flashrnn_forward.cu:150-267. */
int frnn_alt_forward(int function, int dtype, int training, int B, int T, int N, int D,
                     const void* Wx, const void* R, const void* b, const void* s0,
                     void* states, void* cache, void* workspace, size_t workspace_bytes,
                     void* stream);

/* One kernel launch per reverse step: R^T dg_{t+1} of a tile on MFMA, then the adjoint of step t;
 * after the scan the dR GEMM and the bias reduction.
 * Replaces BackwardPass::Run, alternating/flashrnn_backward.cu:267-431. */
int frnn_alt_backward(int function, int dtype, int B, int T, int N, int D,
                      const void* R, const void* b, const void* s0, const void* states,
                      const void* cache, const void* dstates,
                      void* dWx, void* ds0, float* dR, float* db,
                      void* workspace, size_t workspace_bytes, void* stream);

/* ---- options of FlashRNNConfig that change what the kernels compute (flashrnn.py:132-136) ------
 * The reference compiles them in (-DFLASHRNN_FORWARD_CLIPVAL..., -DFLASHRNN_GRADIENT_RECURRENT_CLIPVAL...,
 * flashrnn.py:361-382) and has a separate backward_cut method (fused/flashrnn.cc:248-336,
 * alternating/flashrnn.cc:220-302); here they are run-time arguments of *_opt twins of the four
 * entry points above (opt == NULL or all fields zero: identical to the plain entry point).
 *   forward_clipval > 0:  every new h is clamped to [-v, v] before it is stored and fed back
 *     (lstm_fused_pointwise.cuh:75-80); the backward pass does not see the clamp.  For FRNN_ELMAN the
 *     training forward then fills a gate cache with the unclamped h (sizes: *_cache_bytes_opt), which the
 *     backward call, given the same options, reads for tanh'.
 *   gradient_recurrent_clipval > 0:  in every reverse step the cotangent carried into h_t from
 *     step t+1 is clamped to [-v, v] before the upstream cotangent is added
 *     (lstm_fused_pointwise.cuh:115-121); ds0 itself is not clamped.
 *   gradient_recurrent_cut != 0:  no gradient through R h (FLASHRNNCellFusedBackwardCut,
 *     fused/flashrnn_fused_backward_cut.cu:89-178); dR, db, dWx are still computed.
 * Unlike the reference (which feeds gradient_recurrent_clipval into both clip defines) each
 * option acts on its own. */
typedef struct frnn_options {
  unsigned struct_size;  /* sizeof(frnn_options) of the caller's build: fields are only ever appended, and the library reads
                          * no further than this (a smaller value than the first four fields need is FRNN_E_ARG) */
  float forward_clipval;
  float gradient_recurrent_clipval;
  int gradient_recurrent_cut;
  int recompute;  /* fused backend: no gate cache, see frnn_fused_backward_recompute */
  int batch_stride;  /* fused backend, 0 = B.  The call covers B rows of a batch of batch_stride rows: the state tensors
                      * (s0 and ds0: [S, batch_stride, N, D]; states and dstates: [S, batch_stride, T, N, D]) keep the full
                      * batch's plane stride, and the pointers handed over point at the first row of the range in
                      * plane 0.  Wx, dWx and the gate cache have the batch as their leading axis, so a range of them is
                      * a contiguous block of its own (the gate cache is private to the call that wrote it); dR and db are
                      * the range's own sums.  This is how a batch whose tensors reach 2 GiB runs as several calls that
                      * read and write the caller's tensors in place. */
} frnn_options;

/* Gate-cache size under options: an Elman cell under forward_clipval caches the unclamped h (one value per
 * element, as elman_fused_pointwise.cuh:44-47), without it nothing.  opt == NULL: as the plain queries. */
size_t frnn_fused_cache_bytes_opt(int function, int dtype, int B, int T, int N, int D, const frnn_options* opt);
/* The most batch rows one fused call can take before one of its tensors reaches 2 GiB (FRNN_E_TOO_LARGE), given the plane
 * stride of the state tensors (batch_stride rows; 0: each call's tensors are its own, stride = its B) and whether the
 * gate cache is written (training, and not opt->recompute).  0: not even one row fits at this stride.  The reference
 * has no such limit (fused/flashrnn.cc:68-144 allocates whatever the shape needs). */
int frnn_fused_max_batch(int function, int dtype, int T, int N, int D, int batch_stride, int training, const frnn_options* opt);
size_t frnn_alt_cache_bytes_opt(int function, int dtype, int B, int T, int N, int D, const frnn_options* opt);

int frnn_fused_forward_opt(int function, int dtype, int training, int B, int T, int N, int D,
                           const void* Wx, const void* R, const void* b, const void* s0,
                           void* states, void* cache, void* workspace, size_t workspace_bytes,
                           void* stream, const frnn_options* opt);
int frnn_fused_backward_opt(int function, int dtype, int B, int T, int N, int D,
                            const void* R, const void* b, const void* s0, const void* states,
                            const void* cache, const void* dstates,
                            void* dWx, void* ds0, float* dR, float* db,
                            void* workspace, size_t workspace_bytes, void* stream,
                            const frnn_options* opt);
int frnn_alt_forward_opt(int function, int dtype, int training, int B, int T, int N, int D,
                         const void* Wx, const void* R, const void* b, const void* s0,
                         void* states, void* cache, void* workspace, size_t workspace_bytes,
                         void* stream, const frnn_options* opt);
int frnn_alt_backward_opt(int function, int dtype, int B, int T, int N, int D,
                          const void* R, const void* b, const void* s0, const void* states,
                          const void* cache, const void* dstates,
                          void* dWx, void* ds0, float* dR, float* db,
                          void* workspace, size_t workspace_bytes, void* stream,
                          const frnn_options* opt);

/* ---- recompute mode of the fused backend: training without the gate cache -------------------------------
 * The reference stores the activated gates of every step for the backward pass, unconditionally
 * (fused/flashrnn.cc:97-112, flashrnn_fused_forward.cu:573-644): G_i values per element and step, more than
 * the states themselves.  With opt->recompute != 0 the training forward writes the states only (cache may be
 * null, frnn_fused_cache_bytes_opt is 0), and frnn_fused_backward_recompute, which takes Wx and b in place
 * of the cache, rebuilds the gates of every step from Wx_t, b and R h_(t-1), with h_(t-1) read back from the
 * stored states.  Results equal those of the cached path up to the rounding of the stored states (lstm, gru:
 * the same bits in fp32 storage; slstm: its stabilised gates are rebuilt from the stored, rounded m).
 * Available where R and R^T fit the registers together (frnn_fused_recompute_supported; bf16 / fp16: D = 32, 64,
 * 96, 128, 192, 256, 320, and 384 for the gru; fp32: 32, 64), else FRNN_E_UNSUPPORTED.  For FRNN_ELMAN, which caches nothing, the flag
 * changes nothing.  The workspace size depends on the mode: frnn_fused_workspace_bytes_opt. */
int frnn_fused_recompute_supported(int function, int dtype, int B, int N, int D);
size_t frnn_fused_workspace_bytes_opt(int function, int dtype, int B, int T, int N, int D, int backward,
                                      const frnn_options* opt);
int frnn_fused_backward_recompute(int function, int dtype, int B, int T, int N, int D,
                                  const void* Wx, const void* R, const void* b, const void* s0, const void* states,
                                  const void* dstates, void* dWx, void* ds0, float* dR, float* db,
                                  void* workspace, size_t workspace_bytes, void* stream, const frnn_options* opt);

/* ---- one time step with carried state (inference / decoding) --------------------------------------------
 * Replaces the reference's step kernels (_get_kernel_step, flashrnn.py:957-985, which run the whole-sequence
 * function on a sequence of one; ForwardPass::Iterate, alternating/flashrnn.h:97-101).  One kernel launch,
 * no workspace, nothing cleared, nothing allocated; can be captured into a HIP graph.
 *   Wx_t [B,G_w,N,D], s_in / s_out [S,B,N,D] in the storage type; s_out must not be s_in (ping-pong).
 *   carry: null, or [S,B,N,D] fp32, updated in place: the unrounded state.  The whole-sequence kernels keep
 *     c, n, m (and the h that enters the gate math) in fp32 across time steps and round only what they store;
 *     with a carry a chain of steps does the same and yields the bits of one call over the sequence, without
 *     it every step restarts from the rounded s_in (which is what the reference's step kernel does).  Before
 *     the first step fill it with the initial state converted to fp32. */
int frnn_fused_step(int function, int dtype, int B, int N, int D,
                    const void* Wx_t, const void* R, const void* b, const void* s_in, void* s_out,
                    float* carry, void* stream, const frnn_options* opt);
int frnn_alt_step(int function, int dtype, int B, int N, int D,
                  const void* Wx_t, const void* R, const void* b, const void* s_in, void* s_out,
                  float* carry, void* stream, const frnn_options* opt);

/* Forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose forward allocates its
 * outputs and scratch on every call (fused/flashrnn.cc:97-118).  Same computation and same kernels as
 * frnn_fused_forward_opt, but the workspace (status word + the exchange slots between the workgroups of a
 * head) is a static array in device memory that belongs to the library: 4 MiB per device, held until the
 * process ends (frnn_fused_forward_static_max_bytes()).  The call allocates and frees nothing.  A
 * problem whose frnn_fused_workspace_bytes(..., backward = 0) exceeds that is refused with
 * FRNN_E_WORKSPACE.  All calls on one device share the one array (each call clears the part it uses): two
 * such calls that overlap on a device (different streams or threads) race, so keep them on one stream.
 * The status word cannot be read by the caller; a bounded wait that ran out still shows as NaN in h. */
size_t frnn_fused_forward_static_max_bytes(void);
int frnn_fused_forward_static(int function, int dtype, int training, int B, int T, int N, int D,
                              const void* Wx, const void* R, const void* b, const void* s0,
                              void* states, void* cache, void* stream, const frnn_options* opt);

/* ---- resident decode: the forward kernel stays on the device between tokens ---------------------------------
 * The second half of the reference's step path (flashrnn.py:957-985, alternating/flashrnn.h:97-101), which pays a
 * launch and a reload of R for every token: frnn_fused_decode_open launches the fused forward kernel of the head dim
 * ONCE, on `kernel_stream`; it keeps R in its registers and the state in fp32 registers (as inside a sequence call, so
 * a chain of tokens gives the bits of frnn_fused_forward over the same sequence) and serves one token after the other
 * from a mailbox, a buffer of the caller (frnn_fused_decode_mailbox_bytes, 256-byte aligned, the library clears it
 * in open): a ring of `slots` (2, 4, 8 or 16) inbox and outbox slots of tagged records, one record per element
 * (batch row, head, unit):
 *     inbox  record = the G_w values Wx_t[b, g, n, d] of the element, gate innermost, padded to 1, 2 or 4 values;
 *     outbox record = its S new states; a value of a 16-bit type travels as the dword (tag16 << 16 | bits) with
 *     tag16 = token % 65535 + 1, an fp32 value as two dwords (bits, token + 1).
 *   Offsets inside the buffer: frnn_fused_decode_mailbox_layout.  Any kernel of the caller may write inbox records
 *   (agent-scope stores; a GEMM epilogue, say) and read outbox records; frnn_fused_decode_step is the library's own:
 *   one small launch on `stream` that posts Wx [B, count, G_w, N, D] (count <= slots tokens) and collects s_out
 *   [S, B, count, N, D], taking the token numbers from the mailbox itself, so it can be captured and replayed.
 *   Token t uses slot t % slots; token t + slots may be posted only when token t has been collected.
 * Every wait is bounded: the kernel gives up waiting for a token after `idle_polls` probes (about 0.4 us each) or
 * when frnn_fused_decode_close has set the stop word, or after `max_tokens`, and then ends normally, writing the
 * unrounded state to `carry` ([S,B,N,D] fp32, optional; on entry, if given, it is the unrounded initial state as for
 * frnn_fused_step) and the reason to the control block; the collecting side gives up after FRNN_SPIN_LIMIT probes
 * and writes NaN.  Nothing is allocated.  While a session is open its workgroups occupy their compute units
 * (N * ceil(B / 4) * workgroups-per-head of them; FRNN_E_UNSUPPORTED if they do not fit at once), a device-wide
 * synchronisation waits for the session to end, and `kernel_stream` must not share a hardware queue with `stream`
 * (a runtime maps streams onto a few queues; a post that queues behind the resident kernel is only served when the
 * kernel has idled out).  close orders `stream` behind the end of the resident kernel. */
/* 1 if a kernel launched on `stream` runs while a kernel on `kernel_stream` is still running, 0 if it queues behind it
 * (the runtime maps streams onto a few hardware queues, GPU_MAX_HW_QUEUES, and two streams of one queue run one after
 * the other), negative on error.  Measured, not guessed: a kernel on `kernel_stream` waits up to ~3 ms for a word that a
 * kernel on `stream` sets.  Synchronises both streams; allocates nothing.  frnn_fused_decode_open runs it and refuses
 * a pair that returns 0 (FRNN_E_DEVICE). */
int frnn_streams_overlap(void* stream, void* kernel_stream);
size_t frnn_fused_decode_mailbox_bytes(int function, int dtype, int B, int N, int D, int slots);
/* byte offsets of the inbox and outbox rings and the sizes of one slot of each; the control block is the first 64 ints:
 * [0] status (1: a wait between workgroups ran out), [1] stop word, [2] why the kernel ended (1 wait ran out, 2 idle,
 * 3 stop word, 4 max_tokens), [3] tokens served, [4] 1 if a collecting thread gave up, [9] next token number */
int frnn_fused_decode_mailbox_layout(int function, int dtype, int B, int N, int D, int slots,
                                     size_t* inbox_offset, size_t* inbox_slot_bytes,
                                     size_t* outbox_offset, size_t* outbox_slot_bytes);
int frnn_fused_decode_open(int function, int dtype, int B, int N, int D,
                           const void* R, const void* b, const void* s_in, float* carry,
                           void* mailbox, size_t mailbox_bytes, int slots, int max_tokens, int idle_polls,
                           void* stream, void* kernel_stream, const frnn_options* opt);
int frnn_fused_decode_step(int function, int dtype, int B, int N, int D, int count,
                           const void* Wx, void* s_out, void* mailbox, size_t mailbox_bytes, int slots, void* stream);
int frnn_fused_decode_close(void* mailbox, void* stream, void* kernel_stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHRNN_HIP_H */
