/*
 * C ABI of the MI355X (gfx950) NativeLstm2 forward library (librtn_native_lstm2.so).
 *
 * Plain pointers and sizes only; all data pointers are DEVICE pointers on the
 * current HIP device, `hip_stream` is a hipStream_t (NULL = the default stream).
 * Every entry point only enqueues work on that stream: no device synchronisation
 * (the two *_status queries excepted), no allocation of device memory (scratch comes
 * in through `workspace`; the exception is rocBLAS, which the gradient entries and
 * rtn_lstm_low_mem_fwd call and which may allocate on first use), inputs are never
 * written, outputs are caller-allocated and fully overwritten (the callee does not
 * rely on them being zeroed).
 *
 * The reference has no C ABI of its own for this operator: it generates a C++
 * translation unit per op at run time (returnn/torch/util/native_op.py:83-376)
 * whose body is the op's `c_fw_code` string.  Each function below names the piece
 * of that generated code it stands in for.
 */
#ifndef RTN_NATIVE_LSTM2_H
#define RTN_NATIVE_LSTM2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  The reference signals these through TORCH_CHECK / assert_cmp
 * (returnn/native_op.cpp:60-69, 660); under its -DNDEBUG build the range checks only
 * print.  Here they are hard errors and nothing is enqueued when one is returned. */
#define RTN_OK 0
#define RTN_ERR_SHAPE 1       /* negative or inconsistent T / B / n */
#define RTN_ERR_RANGE 2       /* need 0 <= start < T and step != 0 (returnn/native_op.py:1249-1252) */
#define RTN_ERR_ARG 3         /* null pointer, misaligned pointer, unknown dtype or mode */
#define RTN_ERR_WORKSPACE 4   /* workspace missing or smaller than rtn_native_lstm2_fwd_workspace_bytes() */
#define RTN_ERR_HIP 5         /* a HIP runtime call failed (HANDLE_LAST_ERROR, returnn/native_op.cpp:773-780) */
#define RTN_ERR_UNSUPPORTED 6 /* the requested mode cannot run this shape on this device */
#define RTN_ERR_ABORTED 7     /* reported by rtn_native_lstm2_fwd_status: a bounded in-kernel wait expired */

/* Element type of X, W, y0, Y and H.  The mask i, the cell states c0, C and d are
 * always float32.  F32 is the reference's arithmetic (Ndarray_DEV_DATA casts to float*,
 * returnn/native_op.cpp:647).  BF16 keeps float32 accumulation, gates and cell state. */
#define RTN_DTYPE_F32 0
#define RTN_DTYPE_BF16 1

/* Widths: the matrix-core kernels take n that is a multiple of 32.  Any other n above 32 runs zero-padded to the next
 * multiple of 32 on copies inside the workspace (the size queries include them); the results are those of the
 * unpadded problem, since a padded cell has zero inputs, weights and state.  n up to 32 runs on element-wise kernels. */

/* Execution mode.
 * AUTO:       PERSISTENT when the shape and device allow it, else GRAPH.
 * PERSISTENT: one kernel runs all time steps, all its workgroups on the device together
 *             (a cooperative launch; under stream capture a kernel node that the library
 *             adds to the capturing graph itself, see rtn_native_lstm2_capture_report).  Where the device's registers hold
 *             the recurrent weights (the usual case) every workgroup keeps its slice of W
 *             in registers and the workgroups hand the hidden state over through a ring
 *             of buffers in the workspace that validates itself (a word that still holds
 *             the "not yet written" pattern is read again): no barrier and no flags.
 *             Wider layers fall back to a kernel that keeps W in LDS and separates
 *             the steps with a flag wait.  Every wait is bounded: when one expires the
 *             status word of the workspace is set, the kernel still ends, and NaN is
 *             written into d and the last visited frame of Y (Dy0 and Dc0 in the gradient),
 *             so that a caller who never asks for the status sees non-finite results.
 * GRAPH:      one kernel launch per time step; outside stream capture the launches
 *             are replayed through a library-owned hipGraph, under capture they are
 *             recorded into the caller's graph.
 * STEPWISE:   like GRAPH but always plain launches (no library-owned graph). */
#define RTN_MODE_AUTO 0
#define RTN_MODE_PERSISTENT 1
#define RTN_MODE_GRAPH 2
#define RTN_MODE_STEPWISE 3

/*
 * NativeLstm2 forward.  Replaces the generated op body `c_fw_code`
 * (returnn/native_op.py:1184-1285) together with `lstm_kernel` (:1081-1121), the
 * per-step `affine_raw` GEMM (returnn/native_op.cpp:1032-1067), the `H := X` copy and
 * the zero-initialisation of the outputs done by the generated wrapper
 * (returnn/torch/util/native_op.py:170-184).
 *
 *   X  [T,B,4n]  pre-projected gate inputs; last axis = cell-in | input | forget | output
 *   W  [n,4n]    recurrent weights, same gate order
 *   y0 [B,n]     initial output          c0 [B,n] initial cell state (float32)
 *   i  [T,B]     float32 0/1 mask (right padded batches)
 *   start, step  host ints; step > 0 visits start, start+step, ...; step < 0 visits
 *                T-1-start, T-1-start+step, ... (returnn/native_op.py:1253-1259)
 *   Y  [T,B,n]   output, exactly 0 on masked frames
 *   C  [T,B,n]   cell states (float32), carried over masked frames
 *   H  [T,B,4n]  activated gates, also written on masked frames; frames that are
 *                not visited keep Y = C = 0 and H = X
 *   d  [B,n]     final cell state (float32) = C of the last visited frame; c0 if T == 0
 *
 * All arrays are row-major contiguous and 16-byte aligned.  Returns RTN_OK or an error
 * code; rtn_last_error() describes the last error of the calling thread.
 */
int rtn_native_lstm2_fwd(const void* X, const void* W, const void* y0, const float* c0, const float* i,
                         int32_t start, int32_t step, void* Y, float* C, void* H, float* d, int64_t T,
                         int32_t B, int32_t n, int32_t dtype, int32_t mode, void* workspace,
                         size_t workspace_bytes, void* hip_stream);

/* Bytes of device scratch rtn_native_lstm2_fwd needs for this problem.  Stands in for
 * the op's `device_malloc` of y_prev (returnn/native_op.py:1244, returnn/native_op.cpp:952-960):
 * the caller allocates from its own caching allocator instead.  Calls that overlap in
 * time need distinct workspaces.  Returns 0 on invalid arguments. */
size_t rtn_native_lstm2_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode);

/*
 * rtn_native_lstm2_fwd without a workspace argument, for callers that cannot allocate device memory at the point of the
 * call (code under stream capture that may not grow a pool, tight serving loops, harnesses that forbid allocation).
 * It has no counterpart in the reference.  The scratch lives in a fixed array inside the library's code object
 * (20 MiB per GPU the library runs on, held until the process ends), so the problem's workspace
 * (rtn_native_lstm2_fwd_workspace_bytes) must fit 20 MiB -- that covers widths up to 1024 in both element types with
 * batches up to 128 rows (widths that are not a multiple of 32 need padded copies of all tensors and fit only when
 * small) -- else RTN_ERR_WORKSPACE.  The call allocates nothing on the device and calls
 * no allocating runtime routine: AUTO resolves to PERSISTENT or to plain per-step launches, GRAPH is refused
 * (RTN_ERR_UNSUPPORTED).  Arguments, results and error codes are otherwise those of rtn_native_lstm2_fwd, bit for bit.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU race (keep them on one stream,
 * or order them with events).  The array keeps the previous call's contents; every call re-initialises what it uses.
 * A persistent kernel needs the whole device: do not let a call of this entry overlap in time with persistent calls of
 * the other entries on other streams of the same GPU either (the other entries order their persistent launches among
 * themselves with an event of the library's; this entry creates nothing and joins that order only once the event exists).
 */
int rtn_native_lstm2_fwd_static(const void* X, const void* W, const void* y0, const float* c0, const float* i,
                                int32_t start, int32_t step, void* Y, float* C, void* H, float* d, int64_t T,
                                int32_t B, int32_t n, int32_t dtype, int32_t mode, void* hip_stream);

/* Synchronous check of the last rtn_native_lstm2_fwd that used `workspace`: waits for
 * `hip_stream`, then returns RTN_OK, RTN_ERR_ABORTED (a bounded wait inside the persistent
 * kernel expired, outputs are invalid) or RTN_ERR_HIP.  Stands in for HANDLE_LAST_ERROR
 * after the loop (returnn/native_op.py:1279); optional, for callers that can afford a sync. */
int rtn_native_lstm2_fwd_status(const void* workspace, void* hip_stream);

/*
 * Several independent NativeLstm2 forward calls of one shape (T, B, n, dtype) in one entry: the two
 * directions of a bidirectional layer (one op call with step=+1 and one with step=-1 on the same
 * frames, returnn/tf/layers/rec.py:1229-1270), or the same layer of several streams.  Each element
 * holds the arguments of one rtn_native_lstm2_fwd call and gets exactly that call's results.  When
 * the device can hold the persistent kernel of all of them at once, they run in ONE cooperative
 * launch and hide each other's exchange latency; otherwise they are enqueued back to back.
 * `workspace` holds `count` equal slices, slice k for call k;
 * rtn_native_lstm2_fwd_multi_workspace_bytes(count, ...) gives the total (a slice can be larger than a single
 * call's workspace, because the decomposition may differ when several problems share the device).  The calls must
 * not alias each other's outputs.
 */
typedef struct rtn_lstm2_call {
  const void* X;
  const void* W;
  const void* y0;
  const float* c0;
  const float* i;
  int32_t start;
  int32_t step;
  void* Y;
  float* C;
  void* H;
  float* d;
  /* Row pitch of X and of Y in elements: the distance between the rows of two consecutive (frame, sequence) pairs.
   * 0 = contiguous (4n and n).  A larger pitch lets the calls of a bidirectional layer share arrays the way the reference's
   * caller lays them out (returnn/tf/layers/rec.py:1229-1270 concatenates the two directions' outputs): both directions
   * read their pre-projected gates from one [T*B, 8n] projection (X = base + 0 and base + 4n, ldX = 8n) and write their
   * outputs into one [T, B, 2n] array (Y = base + 0 and base + n, ldY = 2n).  Rows must stay 16-byte aligned. */
  int64_t ldX;
  int64_t ldY;
} rtn_lstm2_call;

int rtn_native_lstm2_fwd_multi(const rtn_lstm2_call* calls, int32_t count, int64_t T, int32_t B, int32_t n,
                               int32_t dtype, int32_t mode, void* workspace, size_t workspace_bytes,
                               void* hip_stream);

size_t rtn_native_lstm2_fwd_multi_workspace_bytes(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype,
                                                  int32_t mode);

/* rtn_native_lstm2_fwd_status over all `count` slices of a multi-call workspace; first failure wins. */
int rtn_native_lstm2_fwd_multi_status(const void* workspace, int32_t count, int64_t T, int32_t B, int32_t n,
                                      int32_t dtype, int32_t mode, void* hip_stream);

/*
 * Measurement aid, not part of the operator: the latency of handing a value from every workgroup to every other
 * one the way the persistent kernel hands over the hidden state (device-scope store, device-scope load until the
 * value has arrived, one workgroup barrier), with 16 workgroups on 16 CUs, 256 bytes each and nothing else going on.
 * Enqueues `rounds` such hand-overs; the caller times the call (events on `hip_stream`) and divides by `rounds`.
 * That time is a lower bound of one time step of any kernel that keeps W spread over several CUs.  `workspace`:
 * at least 16 640 bytes; rtn_native_lstm2_fwd_status(workspace, stream) afterwards tells whether a wait expired.
 * No counterpart in the reference.
 */
int rtn_handover_latency_probe(void* workspace, size_t workspace_bytes, int32_t rounds, void* hip_stream);

/*
 * Measurement aid, not part of the operator: the matrix-core roofline of the plan's own instruction sequence.  Launches,
 * on as many workgroups as the persistent plan for `count` problems of this shape uses, `steps` steps of what that
 * plan's kernel does between the arrival of the hidden state and the pointwise part -- B fragments from LDS, the
 * plan's MFMAs per wavefront against W fragments in registers, the partial tiles through LDS with one barrier, their
 * sum -- with nothing exchanged between workgroups, no streams and no gate arithmetic.  The caller times the call and
 * divides the op's algorithmic flops (8 n^2 per time step and sequence) by it: the rate a kernel of this
 * decomposition could reach at most.  `workspace`: 1 KiB per workgroup of the plan (256 workgroups at most on MI355X).
 * RTN_ERR_UNSUPPORTED for decompositions the probe is not built for.  No counterpart in the reference.
 */
int rtn_mfma_sequence_probe(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t steps, void* workspace,
                            size_t workspace_bytes, void* hip_stream);

/*
 * Measurement aid: the matrix cores alone.  Like rtn_mfma_sequence_probe (same arguments, same grid, same per-wavefront
 * tile sequence with W and the hidden-state fragments in registers), but a step is the MFMAs and nothing else: no LDS
 * round trip of partial tiles, no barrier, no sum.  Launch time over the op's algorithmic flops = the MFMA roofline the
 * plan's tile sequence can reach at most, whatever the rest of a step looks like.  Threads 1 and 2 of every workgroup
 * leave the loop's duration in workspace words 1 and 2 of the workgroup's 1 KiB (float32: shader clocks, ticks of the
 * 100 MHz clock).  Measurement variants for the bf16 plan with 8 tiles per workgroup, chosen by the environment:
 * RTN_LSTM2_PROBE_OTHERS=1..3 puts that many vector instructions behind every MFMA, RTN_LSTM2_PROBE_WAVES=8 deals the
 * MFMAs to two wavefronts per SIMD.  No counterpart in the reference.
 */
int rtn_mfma_issue_probe(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t steps, void* workspace,
                         size_t workspace_bytes, void* hip_stream);

/*
 * NativeLstm2 gradient.  Replaces the generated body `c_bw_code` (returnn/native_op.py:1288-1464) with
 * `lstm_bwd_kernel` (:1123-1180) and its `affine_raw` GEMMs; the arguments are the ones `grad_input_map`
 * (:1071-1077) hands to the gradient op, minus X, which the computation never reads.
 *
 *   W y0 c0 i start step   the forward call's inputs
 *   Y C H                  the forward call's outputs (H = activated gates)
 *   DY [T,B,n]             error signal on Y (values on masked frames are ignored)
 *   Dd [B,n]               error signal on the final cell state d (float32)
 *   DX  [T,B,4n]           out: gradient of X (0 on masked and on unvisited frames)
 *   DW  [n,4n]             out: gradient of W, always float32
 *   Dy0 [B,n]              out: gradient of y0        Dc0 [B,n]  out: gradient of c0 (float32)
 *
 * Element type `dtype` for W y0 Y H DY DX Dy0; c0 C i Dd Dc0 DW are float32.  Where the shape allows (n a multiple of
 * 16, a wavefront's share of 16 rows of W fits its registers, all workgroups fit on the device) ONE persistent
 * cooperative kernel runs all frames: W stays in registers, and the gate derivatives of a frame travel between the
 * workgroups through a ring of 4 frames in the workspace (MFMA operand order, self-validating: a slot is all-ones until
 * written); DX itself is a plain output stream, written once.  Otherwise one launch per visited frame (the MFMA GEMM Dy0 += DX[t'] W^T of the frame processed before,
 * fused with the frame's pointwise part), replayed through a library-owned hipGraph.  The large weight-gradient GEMM
 * (Y^T DX over all frames) is left to rocBLAS, which may allocate its own device workspace on first use.  Under stream
 * capture the kernels (the persistent one as a node of its own, see rtn_native_lstm2_capture_report) and the rocBLAS calls
 * are recorded into the caller's graph (the counterpart of the
 * reference's whole-step graph capture, returnn/torch/util/graph_capture.py); the library's rocBLAS handle (one per host
 * thread and device) has to exist by then: run the entry once outside the capture first, on the capturing thread.  `workspace`: rtn_native_lstm2_bwd_workspace_bytes();
 * rtn_native_lstm2_fwd_status(workspace, stream) reports an expired bounded wait of the persistent kernel.
 */
int rtn_native_lstm2_bwd(const void* W, const void* y0, const float* c0, const float* i, int32_t start, int32_t step,
                         const void* Y, const float* C, const void* H, const void* DY, const float* Dd, void* DX,
                         float* DW, void* Dy0, float* Dc0, int64_t T, int32_t B, int32_t n, int32_t dtype,
                         void* workspace, size_t workspace_bytes, void* hip_stream);

size_t rtn_native_lstm2_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype);

/*
 * Several gradient calls of one shape (T, B, n, dtype) in one entry: the gradient ops of the two directions of a
 * bidirectional layer, which the reference runs as two op calls (the gradient of tf/layers/rec.py:1229-1270).  Element k
 * gives what rtn_native_lstm2_bwd gives for the same arguments, up to float32 rounding (the joint launch may split the
 * work differently, which changes the order of the partial sums).  When the persistent kernel can hold all `count`
 * problems on the device at once (count <= 2) they share one cooperative launch, each workgroup taking more values of k
 * so that every workgroup still has a CU; otherwise the calls are enqueued one after the other.
 * `workspace`: rtn_native_lstm2_bwd_multi_workspace_bytes(); call k uses the k-th equal slice of it, and
 * rtn_native_lstm2_fwd_status(slice k, stream) reports an expired bounded wait of that problem.
 */
typedef struct rtn_lstm2_bwd_call {
  const void* W;
  const void* y0;
  const float* c0;
  const float* i;
  int32_t start;
  int32_t step;
  const void* Y;
  const float* C;
  const void* H;
  const void* DY;
  const float* Dd;
  void* DX;
  float* DW;
  void* Dy0;
  float* Dc0;
  /* Row pitch in elements of Y, DY (rows of n) and DX (rows of 4n), as ldX / ldY of rtn_lstm2_call; 0 = contiguous.  The
   * two directions of a bidirectional layer read the error of one [T, B, 2n] output (DY = base + 0 and base + n,
   * ldDY = 2n) and write their derivatives into one [T*B, 8n] array (DX = base + 0 and base + 4n, ldDX = 8n), from which
   * the gradient of the input projection is then a single product.  H, C and the mask are contiguous. */
  int64_t ldY;
  int64_t ldDY;
  int64_t ldDX;
} rtn_lstm2_bwd_call;

int rtn_native_lstm2_bwd_multi(const rtn_lstm2_bwd_call* calls, int32_t count, int64_t T, int32_t B, int32_t n,
                               int32_t dtype, void* workspace, size_t workspace_bytes, void* hip_stream);

size_t rtn_native_lstm2_bwd_multi_workspace_bytes(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype);

/*
 * Sibling ops of NativeLstm2 on the same kernels (returnn/native_op.py:333-574 and :577-1026), forward pass.  In both,
 * the recurrent input of a frame is the OUTPUT of the frame before -- 0 where that frame was masked -- instead of the
 * last valid output carried over masked frames as in NativeLstm2.
 *
 * LstmGenericBase (c_fw_code :486-523, lstm_kernel :381-429; `NativeLstmCell` of the TF back-end):
 *   Z [T,B,4n] gate inputs, V_h [n,4n], c [B,n] initial cell (float32), i [T,B]  ->  Y [T,B,n], H [T,B,4n] whose first
 *   block holds the CELL STATE and the other three the activated input, forget and output gates, d [B,n] final cell.
 *   No initial output (zero), always all frames in forward order, T > 0.  The reference works in place on Z; here H is
 *   a separate array that must not overlap Z.
 *
 * LstmLowMem (c_fw_code :771-836, lstm_kernel :624-655):
 *   X [T,B,n_in] raw input, W [n_in+n,4n] stacked input and recurrent weights, b [4n], y0, c0 [B,n], i, start, step
 *   ->  Y, C [T,B,n], d [B,n].  start/step as for NativeLstm2 with one difference kept from the reference (:827-833): with
 *   a negative step the loop runs from frame T-start-1 down to frame `start`, not down to frame 0.  Where that visits no
 *   frame (2*start > T-1) the reference returns an unwritten d; here the call is refused with RTN_ERR_RANGE.  Frames the
 *   loop does not visit are zero in Y and C (unwritten in the reference).  The input projection X.W[:n_in] + b is one rocBLAS GEMM over all frames into the
 *   workspace (under stream capture it is recorded like the launches, after one call outside the capture; unlike the reference, the call needs T*B*8n elements of scratch:
 *   the low memory footprint of the reference's variant is not reproduced, only its results).
 */
int rtn_lstm_generic_base_fwd(const void* Z, const void* V_h, const float* c, const float* i, void* Y, void* H, float* d,
                              int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode, void* workspace,
                              size_t workspace_bytes, void* hip_stream);
size_t rtn_lstm_generic_base_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode);

/*
 * Gradient op of LstmGenericBase (c_bw_code returnn/native_op.py:525-574, lstm_bwd_kernel :430-485; inputs as its
 * grad_input_map :374-378): V_h, c, i, the forward results Y and H, DY [T,B,n], Dd [B,n] (float32)  ->  DZ [T,B,4n],
 * DV_h [n,4n] (float32), Dc [B,n] (float32).  Runs on the NativeLstm2 gradient kernels; the reference overwrites H
 * with DZ and DY with a working array, here both inputs are left alone.
 */
int rtn_lstm_generic_base_bwd(const void* V_h, const float* c, const float* i, const void* Y, const void* H, const void* DY,
                              const float* Dd, void* DZ, float* DV_h, float* Dc, int64_t T, int32_t B, int32_t n,
                              int32_t dtype, void* workspace, size_t workspace_bytes, void* hip_stream);
size_t rtn_lstm_generic_base_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n, int32_t dtype);

int rtn_lstm_low_mem_fwd(const void* X, const void* W, const void* b, const void* y0, const float* c0, const float* i,
                         int32_t start, int32_t step, void* Y, float* C, float* d, int64_t T, int32_t B, int32_t n_in,
                         int32_t n, int32_t dtype, int32_t mode, void* workspace, size_t workspace_bytes,
                         void* hip_stream);
size_t rtn_lstm_low_mem_fwd_workspace_bytes(int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype, int32_t mode);

/*
 * Gradient op of LstmLowMem (c_bw_code returnn/native_op.py:864-1026, lstm_bwd_kernel :659-712; inputs as its
 * grad_input_map :619-625): X, W, b, y0, c0, i, start, step, the forward results Y and C, DY [T,B,n], Dd [B,n] (float32)
 *   ->  DX [T,B,n_in], DW [n_in+n,4n] (float32), Db [4n] (float32), Dh [B,n] (error of y0), Dc [B,n] (error of c0, float32).
 * Element type `dtype` for X W b y0 Y DY DX Dh.  The forward pass keeps no gates; where the reference computes them
 * again frame by frame inside its loop (:966-979), here they come from GEMMs over all frames at once (the outputs are
 * known, so that part is no recurrence), the recurrence of the errors runs on the NativeLstm2 gradient kernels over the
 * recurrent rows of W, and DX, the input rows of DW and Db are products and sums over all frames afterwards (rocBLAS).
 * The results are those of the reference's formulas, including what they do on masked frames: the error arriving from
 * the frame processed before is not masked (d_y = DY * mask + d_h, :679), which is the gradient of the forward pass
 * only while no masked frame has valid frames behind it in the recurrence (full-length batches; right-padded batches
 * with step > 0); the reference's own comment (:965) calls the rest unfinished.  Its loop walks back from frame T-1
 * (from frame `start` for step < 0) whatever the stride; where that is not the frame set of the forward pass (the stride
 * does not divide the distance between the two ends) the reference reads outputs that were never written, and the call
 * is refused here with RTN_ERR_RANGE.  Workspace: rtn_lstm_low_mem_bwd_workspace_bytes() (two arrays of T*B*4n elements
 * besides the gradient workspace); rtn_native_lstm2_fwd_status(workspace, stream) reports an expired bounded wait.
 */
int rtn_lstm_low_mem_bwd(const void* X, const void* W, const void* b, const void* y0, const float* c0, const float* i,
                         int32_t start, int32_t step, const void* Y, const float* C, const void* DY, const float* Dd, void* DX,
                         float* DW, float* Db, void* Dh, float* Dc, int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype,
                         void* workspace, size_t workspace_bytes, void* hip_stream);
size_t rtn_lstm_low_mem_bwd_workspace_bytes(int64_t T, int32_t B, int32_t n_in, int32_t n, int32_t dtype);

/*
 * Final output per sequence.  Replaces the caller-side `_lstm_last_output`
 * (returnn/tf/native_op.py:913-929): out[b] = Y[t*, b] for the last visited frame t*
 * (in processing order) with i[t*, b] != 0, else y0[b].  Y, y0, out have element
 * type `dtype`; ldY: row pitch of Y in elements as in rtn_lstm2_call, 0 = n; needs no workspace.
 */
int rtn_native_lstm2_last_output(const void* Y, const void* y0, const float* i, int32_t start, int32_t step,
                                 void* out, int64_t T, int32_t B, int32_t n, int32_t dtype, int64_t ldY, void* hip_stream);

/* Text of the calling thread's last error ("" if none).  Stands in for the message of the
 * exception TORCH_CHECK raises (returnn/native_op.cpp:660). */
const char* rtn_last_error(void);

/* The plan the library would use for this problem, as text
 * ("mode=persistent kernel=mfma_regw mt=2 nt=1 groups=2 wgs_per_group=128 wgs=256 rows_per_group=16
 * launches=1 lds=22176 workspace=...": groups, workgroups and rows per group of one persistent launch, and how many
 * launches in turn take the whole batch); for logs and tests.
 * Counterpart of the reference's compile log next to the .so (returnn/util/native_code_compiler.py:348-352). */
const char* rtn_native_lstm2_describe_plan(int64_t T, int32_t B, int32_t n, int32_t dtype, int32_t mode);

/* The plan used when `count` problems of this shape come in through rtn_native_lstm2_fwd_multi
 * (count = 1: same as rtn_native_lstm2_describe_plan). */
const char* rtn_native_lstm2_describe_multi_plan(int32_t count, int64_t T, int32_t B, int32_t n, int32_t dtype,
                                                 int32_t mode);

/* Library-owned graphs (GRAPH mode; the per-frame launches of the gradient entries): out[0] = graphs kept (at most 8,
 * keyed by shape, element type, plan and device, never by addresses), out[1] = graphs dropped from the cache whose last
 * launch has not completed yet (destroyed at a later call, once it has), out[2] = graphs built so far, out[3] = launches
 * that first wrote another parameter block (other buffers, same shape) into a kept graph, out[4] = graphs destroyed.
 * n_out >= 5.  Replaces nothing in the reference (its ops launch per step, returnn/native_op.py:1254-1277); for tests and
 * for telling a cache that thrashes from one that does not. */
int rtn_graph_cache_stats(int64_t* out, int32_t n_out);

/* What became of the persistent kernels in calls made under stream capture so far (the counterpart of the reference's
 * whole-step graph capture, returnn/torch/util/graph_capture.py:1-80, where its ops are just launches on the capture
 * stream): how many were added to the capturing graph as kernel nodes with the cooperative attribute, how many as
 * ordinary kernel nodes, and, if the runtime refused the cooperative node, which call refused it and with what error.
 * Thread-local text.  RTN_LSTM2_CAPTURE=steps in the environment records per-step launches instead;
 * RTN_LSTM2_CAPTURE_NODE=plain does not try the cooperative attribute. */
const char* rtn_native_lstm2_capture_report(void);

/* The decomposition the last gradient call of the calling thread ran on (kernel, rows per batch group, tiles and
 * wavefronts per workgroup, launches): the gradient entries' counterpart of rtn_native_lstm2_describe_plan, for logs,
 * the benchmark line and tests.  "kernel=bwd_regw_xcd": every batch group on one XCD. */
const char* rtn_native_lstm2_bwd_plan_text(void);

/*
 * The library reads its RTN_LSTM2_* environment variables (experiment and debugging knobs: plan overrides, capture
 * behaviour, wait bounds) once, at its first use, into a snapshot that all later calls plan by; this re-reads them.
 * For programs that change such a variable while running (the tests do).  Thread-safe (a call that runs while another
 * thread re-reads may plan by either snapshot, never by a mixture within one lookup).  The reference has no counterpart: its knobs are Python keyword
 * arguments of make_op (returnn/torch/util/native_op.py:39-57) and one environment variable read at compile time
 * (returnn/util/native_code_compiler.py:63-65).
 */
void rtn_native_lstm2_reload_env(void);

/* ABI version of this header: 13. */
int rtn_native_lstm2_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* RTN_NATIVE_LSTM2_H */
