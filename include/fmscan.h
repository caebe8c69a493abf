/*
 * fmscan.h -- C ABI of libfmscan_hip.so: the Factorization-Memory first-order
 * linear-recurrence scan for AMD MI355X (gfx950), forward and backward.
 *
 *   forward :  h[b,m,d,t] = g[b,m,t] * h[b,m,d,t-1] + (1 - g[b,m,t]) * x[b,d,t]
 *              h[b,m,d,-1] = h0[b,m,d]            (zeros when h0 == NULL)
 *   backward:  delta[t]    = G[t] + g[t+1] * delta[t+1],  delta[L] = first_prop_grad
 *              token_grad  = (1 - g[t]) * delta[t]
 *              gate_grad   = (h[t-1] - x[t]) * delta[t]
 *
 * Every pointer is a device pointer on the GPU that is current when the call
 * is made; all tensors are dense, row-major, sequence (L) innermost. The
 * library owns no memory and keeps no state between calls: the caller
 * allocates inputs, outputs and the optional workspace, the calls enqueue
 * kernels on `stream` (a hipStream_t, NULL = the default stream) and return
 * without waiting.
 *
 * Workspace. With very few rows (B*M*D < 32) and long sequences a row is
 * cut into segments that are scanned side by side; the carry between segments
 * goes through `workspace` (two floats per segment, written by a first pass).
 * fmscan_workspace_bytes() tells how much a call can use; a NULL or smaller
 * workspace makes the call scan every row in one piece (same results up to
 * rounding, fewer compute units busy). Calls that run concurrently need
 * separate workspaces.
 *
 * These entry points stand where the reference's two extension functions
 * stand (reference fm/scan/fm_scan.cuh:344-358 `fm_scan_forward`, :361-381
 * `fm_scan_backward`, with the launcher :248-331 and dtype dispatch :333-342
 * behind them); the torch::Tensor arguments of those functions become plain
 * pointers plus the four sizes the launcher reads from `out.sizes()` (:265-269).
 *
 * Return value of every int function: 0 on success, a negative FMSCAN_E_*
 * code for a rejected argument (nothing was launched), a positive hipError_t
 * when the HIP runtime refused the launch. fmscan_last_error() gives the text.
 */
#ifndef FMSCAN_H_
#define FMSCAN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMSCAN_ABI_VERSION 7

/* element type of every tensor in one call (reference fm_scan.cuh:333-342) */
#define FMSCAN_DTYPE_F32  0
#define FMSCAN_DTYPE_F16  1
#define FMSCAN_DTYPE_BF16 2

/* flags */
#define FMSCAN_FLAG_PLAIN        0x1u /* core operator h_t = g_t h_{t-1} + x_t: no (1-g) input
                                         scaling; backward: token_grad = delta,
                                         gate_grad = h[t-1] * delta (input_tokens unused) */
#define FMSCAN_FLAG_WAVES_SHIFT  8    /* bits 8..11: waves cooperating on one row (1,2,4,8);
                                         0 = let the library choose */
#define FMSCAN_FLAG_WAVES_MASK   0xF00u
#define FMSCAN_FLAG_BLOCKS_SHIFT 12   /* bits 12..15: cap on the blocks a compute unit holds at a
                                         time (1..15); 0 = let the library choose */
#define FMSCAN_FLAG_BLOCKS_MASK  0xF000u
#define FMSCAN_FLAG_DEPTH_SHIFT  16   /* bits 16..19: tiles whose loads a wave keeps in flight
                                         ahead of the one it scans (2 or 4); 0 = library's choice */
#define FMSCAN_FLAG_DEPTH_MASK   0xF0000u
#define FMSCAN_FLAG_SEGMENTS_SHIFT 20 /* bits 20..27: segments a row is cut into (2..255, needs the
                                         workspace); 1 = never cut; 0 = library's choice */
#define FMSCAN_FLAG_SEGMENTS_MASK 0xFF00000u
/* With none of the four choices above made by the caller, fmscan_forward, fmscan_forward_static and
 * fmscan_backward put rows of at most 1 KiB several to a wave (a kernel of its own, a segmented wave scan);
 * any of them set selects the general kernels, which give a wave one row at a time. Results agree to
 * float32 rounding. The layer's calls (fmscan_forward_normed, fmscan_readout_forward, fmscan_readout_backward,
 * fmscan_readout_dot) do the same by themselves for rows of at most 256 bytes (512 for the read-out's two)
 * when there is enough work for it; their results do not change shape. */

/* error codes (negative returns) */
#define FMSCAN_E_NULL      (-1) /* a required pointer is NULL */
#define FMSCAN_E_SHAPE     (-2) /* B, M, D or L is < 1, or a size overflows */
#define FMSCAN_E_DTYPE     (-3) /* dtype is not one of FMSCAN_DTYPE_* */
#define FMSCAN_E_FLAGS     (-4) /* unknown flag bit or unsupported waves-per-row value */
#define FMSCAN_E_ALIAS     (-5) /* an output overlaps an input it must not overlap */
#define FMSCAN_E_WORKSPACE (-6) /* segments were requested and the workspace is missing or small */
#define FMSCAN_E_UNALIGNED (-7) /* this entry point needs 16-byte aligned pointers and rows */

/* Version of this interface; equals FMSCAN_ABI_VERSION of the header the
 * library was built from. No counterpart in the reference (its extension is
 * JIT-built from source at import, fm/scan/fm_scan.py:18-33). */
int fmscan_abi_version(void);

/* Hash of the sources and compiler flags the library was built from (16 hex digits), so
 * that a loader can tell a library older than its sources. No counterpart in the
 * reference, which compiles its source at every import (fm/scan/fm_scan.py:18-33). */
const char* fmscan_build_id(void);

/* Text of the last error raised on the calling thread ("" if none).
 * Replaces the c10::Error text of the reference's TORCH_CHECKs
 * (fm/scan/fm_scan.cuh:329,341,346-354,367-378). */
const char* fmscan_last_error(void);

/* Bytes of workspace fmscan_forward / fmscan_backward can use for this problem (0 when
 * rows are never cut). No counterpart in the reference, whose kernel gives one block a
 * whole row (fm/scan/fm_scan.cuh:62-64,84). */
size_t fmscan_workspace_bytes(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags);

/*
 * Forward scan. Replaces fm_scan_forward (reference fm/scan/fm_scan.cuh:344-358)
 * and the forward instantiation of its kernel (:42-218 with reverse=false,
 * backward=false).
 *   gates          (B, M, L)     in
 *   tokens         (B, D, L)     in
 *   initial_state  (B, M, D)     in, may be NULL (= zeros)
 *   out            (B, M, D, L)  out; must not overlap gates or tokens
 * Any L >= 1 is accepted (the reference accepts powers of two in 32..131072,
 * fm_scan.cuh:275-329); aligned 16-byte vector access is used when the pointers and
 * L * sizeof(element) are multiples of 16; otherwise 16-byte accesses at the alignment of an element,
 * and element access for the ragged end of a row (about 0.6 of the aligned rate).
 */
int fmscan_forward(const void* gates, const void* tokens, const void* initial_state,
                   void* out,
                   int64_t B, int64_t M, int64_t D, int64_t L,
                   int dtype, unsigned flags,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * fmscan_forward for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid it) and so cannot bring the workspace
 * that cut rows need: same arguments and results as fmscan_forward, with the segment pairs
 * in device memory that the library itself holds, a static array of FMSCAN_STATIC_PAIRS
 * pairs (64 KiB) on every GPU the call has been used on, kept until the process ends. It
 * has no counterpart in the reference (whose kernel gives a whole row to one block and
 * needs no workspace, fm/scan/fm_scan.cuh:62-64,84). The call allocates nothing. Every
 * automatic cut fits (fewer than 32 rows, at most 255 segments each); a requested cut
 * (FMSCAN_FLAG_SEGMENTS) of more than FMSCAN_STATIC_PAIRS segments in total is rejected
 * with FMSCAN_E_WORKSPACE. All calls on one GPU share the array: calls whose rows are cut
 * must not overlap in time on the same GPU (different streams, different threads), or
 * they overwrite each other's pairs. Nothing in the array needs clearing between calls:
 * every pair a call reads, that call has written first. The first call on a GPU looks up
 * the array's address; make that call before capturing a graph.
 */
#define FMSCAN_STATIC_PAIRS 8192
int fmscan_forward_static(const void* gates, const void* tokens, const void* initial_state,
                          void* out,
                          int64_t B, int64_t M, int64_t D, int64_t L,
                          int dtype, unsigned flags, void* stream);

/*
 * Backward scan. Replaces fm_scan_backward (reference fm/scan/fm_scan.cuh:361-381)
 * and the backward instantiation of its kernel (:42-218 with reverse=true,
 * backward=true; gate shift :103-108, epilogues :184-185 and :188-208).
 *   gates            (B, M, L)     in
 *   out_grad         (B, M, D, L)  in   dL/dh
 *   first_prop_grad  (B, M, D)     in, may be NULL (= zeros): gradient flowing in
 *                                       from beyond the last step (:360)
 *   token_grad_out   (B, M, D, L)  out  (1 - g) * delta per (m, d)
 *   cached_output    (B, M, D, L)  in   h as the forward call wrote it for these gates, tokens
 *                    and initial state. With FMSCAN_FLAG_PLAIN every element is read (h[t-1]
 *                    enters the gate gradient, as in the reference kernel, :189-197). Without the
 *                    flag it is read at one position per wave and tile only (the element just
 *                    before the wave's part of the tile, and h[0]); the states in between are
 *                    made again in float32 from gates and input_tokens. A buffer that is not the
 *                    forward output for these inputs therefore gives a gate gradient the
 *                    reference kernel would not give for it; the other outputs do not depend on it.
 *   input_tokens     (B, D, L)     in   (ignored with FMSCAN_FLAG_PLAIN)
 *   gate_grad_out    (B, M, D, L)  out  (h[t-1] - x[t]) * delta per (m, d)
 *   initial_state    (B, M, D)     in, may be NULL: h[-1] used by gate_grad at t = 0.
 *                    NULL reproduces the reference kernel, which reads its own
 *                    `initial_state` argument there and is handed first_prop_grad
 *                    (:196 with :380), i.e. h[-1] := first_prop_grad (zeros if that
 *                    is NULL too). Pass the forward call's initial_state to get the
 *                    mathematically exact gate gradient at t = 0.
 *   initial_state_grad (B, M, D)   out, may be NULL: dL/d initial_state = g[0] * delta[0].
 *                    The reference leaves this gradient unconnected
 *                    (fm/scan/fm_scan.py:80-81); its per-timestep PyTorch path
 *                    (fm/scan/fm_pytorch.py) yields it through autograd.
 * Outputs must not overlap any input or each other.
 */
int fmscan_backward(const void* gates, const void* out_grad, const void* first_prop_grad,
                    void* token_grad_out,
                    const void* cached_output, const void* input_tokens,
                    void* gate_grad_out,
                    const void* initial_state, void* initial_state_grad,
                    int64_t B, int64_t M, int64_t D, int64_t L,
                    int dtype, unsigned flags,
                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward scan with the two sums of FM_Scan.backward inside (reference
 * fm/scan/fm_scan.py:70-78: d_gates = gateGradOut.sum(dim=2), d_tokens =
 * tokenGradOut.sum(dim=1); the reference's kernel writes both (B, M, D, L) tensors in
 * full, fm/scan/fm_scan.cuh:200-207, and names the fused form as a TODO). Meant for
 * M > 1 and D > 1; the per-pair tensors are never written.
 *   token_grad         (B, D, L)     out, element dtype: sum over m of (1 - g) * delta
 *   gate_grad_partial  (B, M, G, L)  out, float32, G = fmscan_reduced_groups(B, D): the sum of
 *                      (h[t-1] - x[t]) * delta over each group of 8 consecutive d (of 4 where 8
 *                      would leave too few blocks for the GPU: small B * D);
 *                      d_gates[b,m,t] is the sum of the G partials (one more small pass
 *                      for the caller; sums are accumulated in float32 throughout)
 * Other arguments as fmscan_backward, cached_output included: without FMSCAN_FLAG_PLAIN it
 * must be the forward call's output for these gates and tokens and is read at one position per
 * row and tile (the element before the tile, and h[0]); the rest is made again from gates and
 * input_tokens. Needs 16-byte aligned pointers and
 * L * sizeof(element) % 16 == 0 (FMSCAN_E_UNALIGNED otherwise: use fmscan_backward);
 * flags: only FMSCAN_FLAG_PLAIN.
 */
int64_t fmscan_reduced_groups(int64_t B, int64_t D);
/* out[r, t] = sum over g of partial[r, g, t] for float32 partial (rows, G, L), rounded once to
 * the call's dtype: d_gates (B, M, L) from gate_grad_partial with rows = B * M (the reference's
 * torch.sum at fm/scan/fm_scan.py:76). Groups are added in their order: deterministic. */
int fmscan_sum_groups(const float* partial, int64_t G, void* out, int64_t rows, int64_t L, int dtype,
                      void* stream);
int fmscan_backward_reduced(const void* gates, const void* out_grad, const void* first_prop_grad,
                            void* token_grad,
                            const void* cached_output, const void* input_tokens,
                            float* gate_grad_partial,
                            const void* initial_state, void* initial_state_grad,
                            int64_t B, int64_t M, int64_t D, int64_t L,
                            int dtype, unsigned flags, void* stream);

/*
 * fmscan_backward_reduced for a scan inside the Factorization-Memory layer (reference
 * fm/scan/fm_scan.py:121-131 differentiated as one piece): the gradient arriving at the
 * scanned states is not passed as a (B, M, D, L) tensor but made inside the kernel,
 *   G[b,m,d,t] = coef_out[b,m,t] * out_grad[b,d,t] - coef_self[b,m,t] * states_n[b,m,d,t],
 * which is the gradient of the RMS norm and read-out (fmscan_readout_backward without
 * ext_grad) when coef_out = inv_rms * read and coef_self = inv_rms * read * q / D, and of
 * the read-out alone when coef_out = read, coef_self = 0 and states_n = cached_output.
 *   states_n   (B, M, D, L)  the normalised states      coef_out, coef_self  (B, M, L) float32
 *   out_grad   (B, D, L)     gradient of the layer's output, time last
 * states_n and out_grad of the call's dtype. cached_output, when given, is the forward
 * call's output for these gates and tokens, read as fmscan_backward_reduced reads it (one
 * position per row and tile). It may be NULL when rms ((B, M, L) float32, 1 / inv_rms:
 * fmscan_readout_dot writes it) is given: the scanned states are then taken back from the
 * normalised ones, states_n * rms (every element of states_n is read anyway), and the layer
 * need not keep them (the reference keeps them for autograd, fm/scan/fm_scan.py:53-55).
 * Everything else, and the limits, as fmscan_backward_reduced.
 */
int fmscan_backward_layer(const void* gates, const void* states_n,
                          const float* coef_out, const float* coef_self, const void* out_grad,
                          const void* first_prop_grad, void* token_grad,
                          const void* cached_output, const float* rms,
                          const void* input_tokens, float* gate_grad_partial,
                          const void* initial_state, void* initial_state_grad,
                          int64_t B, int64_t M, int64_t D, int64_t L,
                          int dtype, unsigned flags, void* stream);

/*
 * fmscan_backward_reduced and fmscan_backward_layer for problems with few batch elements and
 * long rows. Their kernel gives a block to every (b, group of 4 or 8 consecutive d) and walks
 * the row from its end to its start, so B * ceil(D / 4) blocks are all the parallelism it has;
 * below 512 of them part of the GPU stands idle (the reference's kernel has a block per row,
 * fm/scan/fm_scan.cuh:221-342, and does not know the situation). With split > 1 (a divisor of
 * M, M / split >= 4) the M slots of a batch element are dealt to `split` blocks; the token
 * gradient, a sum over all slots, is then left as float32 partial sums
 *   token_grad_partial  (B, D, split, L)  out, float32
 * for fmscan_sum_groups (rows = B * D, G = split), which adds them in their order and rounds
 * once: deterministic like the rest (these two calls write it for split = 1 as well). gate_grad_partial
 * is (B, M, G, L) with G = fmscan_reduced_groups(B * split, D). fmscan_reduced_split(B, M, D): the split
 * these calls should be given for a shape (1: use the calls above; 0 for a shape that is none).
 * Both can also cut the rows into `segments` pieces (1 <= segments <= 255, at
 * most one per tile of 256 float32 / 512 16-bit elements; without FMSCAN_FLAG_PLAIN only), each piece a
 * block of its own, in two passes: the first runs the kernel without accumulating or storing any gradient
 * and leaves every segment's step pair (its gate product and what leaves it when nothing enters) in
 *   workspace  B * M * D * segments * 8 bytes, 8-byte aligned (FMSCAN_E_WORKSPACE otherwise),
 * the second is the kernel proper, started inside the row with what those pairs give. It reads states_n
 * (out_grad) twice, which pays where the blocks are few. fmscan_reduced_plan(B, M, D, L, dtype, &split,
 * &segments): the split and the number of segments the library would use for a shape (1 and 1: call
 * fmscan_backward_layer or fmscan_backward_reduced); returns 0, or an error code with both left 0.
 * No counterpart in the reference; everything else as the two calls above.
 */
int64_t fmscan_reduced_split(int64_t B, int64_t M, int64_t D);
/* 1 when fmscan_backward_reduced (split and cut as fmscan_reduced_plan below says) is expected to be at
 * least as fast as fmscan_backward followed by the two sums, 0 when even that leaves too few blocks
 * (very few batch elements with few slots and channels, rows too short to cut) and for rows of up to
 * 256 bytes, where fmscan_backward puts several rows into a wave and this kernel
 * leaves most lanes idle. */
int fmscan_reduced_pays(int64_t B, int64_t M, int64_t D, int64_t L, int dtype);
/* fmscan_backward_reduced for short rows: rows of whole 16-byte vectors up to 256 bytes, which
 * fmscan_backward_reduced gives a wave instruction each (most lanes idle). Several rows share a wave, a wave
 * takes one batch element and a tile of rows d and walks the M slots: token_grad (B, D, L) is complete,
 * gate_grad_partial is (B, M, G, L) float32 with G = fmscan_reduced_packed_groups(B, M, D, L, dtype), to be
 * added by fmscan_sum_groups. That query returns 0 where the call does not apply (longer or unaligned rows,
 * fewer than 512 (b, tile) pairs): then the call returns FMSCAN_E_SHAPE. Arguments, flags (FMSCAN_FLAG_PLAIN
 * only) and results otherwise as fmscan_backward_reduced; results agree with it to float32 rounding.
 * No counterpart in the reference (fm_scan.py:70-78 writes two (B, M, D, L) tensors and sums them). */
int64_t fmscan_reduced_packed_groups(int64_t B, int64_t M, int64_t D, int64_t L, int dtype);
int fmscan_backward_reduced_packed(const void* gates, const void* out_grad, const void* first_prop_grad,
                                   void* token_grad, const void* cached_output, const void* input_tokens,
                                   float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                                   int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                                   void* stream);
/* The same for the layer's form: arguments and results as fmscan_backward_layer (both of its forms: the
 * saved states in cached_output, or NULL there and rms), gate_grad_partial as above. No counterpart in the
 * reference. */
int fmscan_backward_layer_packed(const void* gates, const void* states_n, const float* coef_out,
                                 const float* coef_self, const void* out_grad, const void* first_prop_grad,
                                 void* token_grad, const void* cached_output, const float* rms,
                                 const void* input_tokens, float* gate_grad_partial, const void* initial_state,
                                 void* initial_state_grad, int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                                 unsigned flags, void* stream);
int fmscan_backward_reduced_split(const void* gates, const void* out_grad, const void* first_prop_grad,
                                  float* token_grad_partial,
                                  const void* cached_output, const void* input_tokens,
                                  float* gate_grad_partial,
                                  const void* initial_state, void* initial_state_grad,
                                  int64_t B, int64_t M, int64_t D, int64_t L, int64_t split,
                                  int64_t segments, void* workspace, size_t workspace_bytes,
                                  int dtype, unsigned flags, void* stream);
int fmscan_backward_layer_split(const void* gates, const void* states_n,
                                const float* coef_out, const float* coef_self, const void* out_grad,
                                const void* first_prop_grad, float* token_grad_partial,
                                const void* cached_output, const float* rms,
                                const void* input_tokens, float* gate_grad_partial,
                                const void* initial_state, void* initial_state_grad,
                                int64_t B, int64_t M, int64_t D, int64_t L, int64_t split,
                                int64_t segments, void* workspace, size_t workspace_bytes,
                                int dtype, unsigned flags, void* stream);
int fmscan_reduced_plan(int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                               int64_t* split, int64_t* segments);

/*
 * The read-out of the Factorization-Memory layer (reference fm/scan/fm_scan.py:124-131,
 * inside fm_memory): RMS norm of the scanned states over the D axis of every memory slot
 *   inv_rms[b,m,t] = rsqrt(mean_d states[b,m,d,t]^2 + eps)            (:126)
 *   normalised     = states * inv_rms                                  (:127)
 * and the output projection over the M slots
 *   output[b,d,t]  = sum_m read[b,m,t] * normalised[b,m,d,t]           (:130-131,
 * einsum 'blm,bmdl->bld' with read = (alpha * output_scale) laid out (B, M, L); the
 * caller transposes output to the reference's (B, L, D)). The reference leaves these to
 * five PyTorch operations over (B, M, D, L) tensors and to autograd; the four calls
 * below are their forward and backward with fp32 arithmetic and one rounding per
 * stored value. Every tensor is dense with L innermost, of the call's dtype unless
 * marked float32. Any L; 16-byte aligned pointers with L * sizeof(element) % 16 == 0
 * take the vector path. B * M * ceil(L / tile) must be < 2^31 (tile = 256 float32 /
 * 512 16-bit elements) and D < 2^20.
 *
 * fmscan_readout_inv_rms:   inv_rms (B, M, L) float32 out.
 * fmscan_readout_forward:   inv_rms NULL = no norm (mem_norm=False, :125): states_out
 *                           is then ignored and the read-out sees `states`; otherwise
 *                           states_out (B, M, D, L) receives the normalised states (it
 *                           may be the same buffer as `states`), and the read-out uses
 *                           the stored (rounded) values as the reference does.
 * fmscan_readout_dot:       q[b,m,t] = sum_d out_grad[b,d,t] * states_n[b,m,d,t]
 *                           (float32; it is the gradient of `read`) and, when ext_grad
 *                           (a gradient arriving at the returned memory states,
 *                           (B, M, D, L)) is not NULL, qe = sum_d ext_grad * states_n.
 *                           With coef_out and coef_self ((B, M, L), float32)
 *                           not NULL it also writes what fmscan_backward_layer takes:
 *                           coef_out = inv_rms * read, coef_self = coef_out * q / D
 *                           (inv_rms NULL: coef_out = read, coef_self = 0), and with rms_out
 *                           ((B, M, L), float32) not NULL, rms_out = 1 / inv_rms.
 * fmscan_readout_backward:  state_grad (B, M, D, L) = gradient of the scanned states:
 *                           dn = read * out_grad (+ ext_grad);
 *                           with the norm  inv_rms * (dn - states_n * (read*q + qe) / D),
 *                           without it     dn  (states_n, inv_rms, q, qe unused, may be NULL).
 * Return values as for the scan calls.
 */
int fmscan_readout_inv_rms(const void* states, float* inv_rms,
                           int64_t B, int64_t M, int64_t D, int64_t L, int dtype, float eps,
                           void* stream);
int fmscan_readout_forward(const void* states, const float* inv_rms, const void* read,
                           void* states_out, void* output,
                           int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream);
int fmscan_readout_dot(const void* states_n, const void* out_grad, const void* ext_grad,
                       float* q, float* qe,
                       const float* inv_rms, const void* read, float* coef_out, float* coef_self,
                       float* rms_out,
                       int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream);
int fmscan_readout_backward(const void* states_n, const float* inv_rms, const void* read,
                            const void* out_grad, const void* ext_grad,
                            const float* q, const float* qe, void* state_grad,
                            int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream);

/*
 * Forward scan and RMS norm in one call (reference fm/scan/fm_scan.py:121-127 inside
 * fm_memory: fm_scan, then states * rsqrt(mean(states^2, dim=2) + eps)): what fmscan_forward,
 * fmscan_readout_inv_rms and the scaling half of fmscan_readout_forward compute one after the
 * other, without the scanned states ever reaching memory. A block holds all D rows of a
 * memory slot in registers, hence D <= fmscan_forward_normed_max_d() (FMSCAN_E_SHAPE beyond:
 * use the three calls), and it needs 16-byte aligned pointers with
 * L * sizeof(element) % 16 == 0 (FMSCAN_E_UNALIGNED otherwise).
 *   gates (B, M, L), tokens (B, D, L), initial_state (B, M, D) or NULL    in
 *   states_n (B, M, D, L)   out: the normalised states (each state is rounded to the call's
 *                           dtype before it enters the norm, as a stored state would be)
 *   inv_rms  (B, M, L)      out, float32
 * The read-out over the slots is then fmscan_readout_forward(states_n, NULL, read, NULL, output).
 */
int64_t fmscan_forward_normed_max_d(void);
/* 1 when this call (or fmscan_forward_sumsq below, for larger D) is expected to be the faster way to
 * the normalised states for a shape, 0 when the three calls are: a block of these kernels is a slot
 * (or 128 rows of one) for the whole length of the sequence, and few batch elements with few slots
 * leave most of the GPU idle. No counterpart in the reference. */
int fmscan_forward_normed_pays(int64_t B, int64_t M, int64_t D);
int fmscan_forward_normed(const void* gates, const void* tokens, const void* initial_state,
                          void* states_n, float* inv_rms,
                          int64_t B, int64_t M, int64_t D, int64_t L,
                          int dtype, float eps, void* stream);
/* The same with every slot's sequence cut into `segments` pieces (1 <= segments <= 255, at most one per
 * tile of 256 float32 / 512 16-bit elements), each piece a block of its own: for few slots and long rows,
 * where a block per slot leaves most of the GPU idle. Two passes, like fmscan_forward's cut rows: the
 * first reduces every segment of every row to its step pair (it reads only gates and tokens) into
 *   workspace  B * M * D * segments * 8 bytes, 8-byte aligned (FMSCAN_E_WORKSPACE otherwise),
 * the second is the kernel of fmscan_forward_normed started inside the row with the state those pairs
 * give. Results agree with the uncut call to rounding. fmscan_forward_normed_segments: the number of
 * segments the library would cut a shape into (1: call fmscan_forward_normed; 0: a shape this kernel
 * does not take). No counterpart in the reference. */
int64_t fmscan_forward_normed_segments(int64_t B, int64_t M, int64_t D, int64_t L, int dtype);
int fmscan_forward_normed_cut(const void* gates, const void* tokens, const void* initial_state,
                              void* states_n, float* inv_rms,
                              int64_t B, int64_t M, int64_t D, int64_t L,
                              int dtype, float eps,
                              int64_t segments, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same for any D, in two steps: fmscan_forward_sumsq is fmscan_forward (16-byte aligned rows only,
 * FMSCAN_E_UNALIGNED otherwise) that also leaves the sums of squares of the states it stores (rounded to
 * the call's dtype first, as fmscan_readout_inv_rms reads them) over blocks of 128 consecutive d:
 *   sumsq_partial (B, M, G, L) float32, G = fmscan_sumsq_groups(D),
 * so that the norm (reference fm/scan/fm_scan.py:125-126) needs no pass over the states of its own;
 * fmscan_sumsq_finish turns the partial sums into inv_rms (B, M, L) float32 =
 * rsqrt(sum_g partial / D + eps). fmscan_readout_forward(states, inv_rms, ...) follows.
 */
int64_t fmscan_sumsq_groups(int64_t D);
int fmscan_forward_sumsq(const void* gates, const void* tokens, const void* initial_state,
                         void* states, float* sumsq_partial,
                         int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream);
int fmscan_sumsq_finish(const float* sumsq_partial, int64_t G, float* inv_rms,
                        int64_t B, int64_t M, int64_t D, int64_t L, float eps, void* stream);

/*
 * The layer's small tensors (reference fm/scan/fm_scan.py:116,118-119,130 and their
 * gradients): alpha (B, L, M), update_scale and output_scale (B, L, 1), all of the call's
 * dtype.
 * fmscan_layer_prepare:  gates[b,m,t] = 1 - alpha[b,t,m] * update_scale[b,t] and
 *                        read[b,m,t] = alpha[b,t,m] * output_scale[b,t], both (B, M, L).
 * fmscan_layer_finish:   from the gradient of gates, given as G float32 partials
 *                        (B, M, G, L) to be summed (what fmscan_backward_reduced and
 *                        fmscan_backward_layer write; G = 1 for a plain (B, M, L) gradient),
 *                        and of read (B, M, L) float32 (q of fmscan_readout_dot):
 *                        alpha_grad = read_grad * output_scale - gate_grad * update_scale,
 *                        update_scale_grad = -sum_m gate_grad * alpha,
 *                        output_scale_grad = sum_m read_grad * alpha.
 */
int fmscan_layer_prepare(const void* alpha, const void* update_scale, const void* output_scale,
                         void* gates, void* read,
                         int64_t B, int64_t L, int64_t M, int dtype, void* stream);
int fmscan_layer_finish(const float* gate_grad_partial, int64_t G, const float* read_grad,
                        const void* alpha, const void* update_scale, const void* output_scale,
                        void* alpha_grad, void* update_scale_grad, void* output_scale_grad,
                        int64_t B, int64_t L, int64_t M, int dtype, void* stream);

/*
 * dst[b, c, r] = src[b, r, c] for dense (B, R, C) -> (B, C, R): what fm_memory does to its
 * (B, L, *) arguments and to its output with transpose(1, 2).contiguous() (reference
 * fm/scan/fm_scan.py:117-118,131). element_size 2 or 4; src and dst must not overlap.
 */
int fmscan_swap_last_two(const void* src, void* dst, int64_t B, int64_t R, int64_t C,
                         int element_size, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FMSCAN_H_ */
