/*
 * libblr - structured-linear forward kernels for AMD MI355X (gfx950).
 *
 * C ABI of the shared library.  Every entry point
 *   - takes plain device pointers and sizes (no framework types),
 *   - only enqueues work on the HIP stream it is given (NULL = the null stream); it never
 *     synchronises, never allocates and never frees device memory,
 *   - borrows every buffer for the duration of the enqueued work,
 *   - returns 0 on success or a negative blr_status; the text of the last failure on the
 *     calling thread is available from blr_last_error().
 *
 * Row-major everywhere.  "M" is the number of token rows (batch * sequence).  x may be a
 * strided view: row m starts at x + m * ldx elements.  Weights must be contiguous.
 * dtype selects the element type of x, of the floating-point weights and of out.
 *
 * Each entry point names the function of the reference implementation
 * (pabillam/mem-efficient-blr) whose arithmetic and operand layout it reproduces.
 */
#ifndef BLR_H
#define BLR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  BLR_OK = 0,
  BLR_ERR_BAD_ARG = -1,       /* null pointer, non-positive size, unknown enum value        */
  BLR_ERR_BAD_SHAPE = -2,     /* in_f % b, out_f % b, rank % b ... violated                  */
  BLR_ERR_WORKSPACE = -3,     /* workspace missing or smaller than blr_*_workspace_bytes()  */
  BLR_ERR_UNSUPPORTED = -4,   /* combination not implemented (e.g. decode algo with fp32)   */
  BLR_ERR_LAUNCH = -5,        /* the HIP runtime refused a launch                            */
  BLR_ERR_NO_DEVICE = -6,
  BLR_ERR_TIMEOUT = -7        /* a bounded wait inside a kernel gave up (blr_workspace_status)  */
} blr_status;

typedef enum { BLR_F16 = 0, BLR_BF16 = 1, BLR_F32 = 2 } blr_dtype;

/* BLAST U factor: (b, r, q) for the partial/full function names, (b, q, r) for the bmm names
 * (reference models/wrappers.py:151-159).                                                    */
typedef enum { BLR_U_RQ = 0, BLR_U_QR = 1 } blr_u_layout;

/* BLAST S factor: (b1=j, b2=i, r) for partial/full names, (r, b2=i, b1=j) for bmm names,
 * (b2=i, b1=j, r) for the torch baseline layout (reference layer.py:193-200).               */
typedef enum { BLR_S_JIR = 0, BLR_S_RIJ = 1, BLR_S_IJR = 2 } blr_s_layout;

/* Which kernel family serves a call.  AUTO picks STREAM for M <= 16 of f16 / bf16 (HBM-bound) and TILED otherwise. */
typedef enum {
  BLR_ALGO_AUTO = 0,
  BLR_ALGO_STREAM = 1,        /* the few-row kernels, M <= 16, f16/bf16: one to three launches chosen by row count and shape (one or two
                                 at M = 1, three on the matrix cores at 2..16 rows; a single persistent launch for what those decline) */
  BLR_ALGO_TILED = 2,         /* up to 128 rows: the three-launch few-row kernels over tiles of 16 rows; above: MFMA tiled GEMMs with the
                                 rank-space intermediates in the workspace (narrow blocks: fused launches that keep Y and / or Z on chip) */
  BLR_ALGO_FUSED = 3,         /* BLAST: x V and the mix in one launch, Y = x V only ever in LDS; then the batched GEMM with U.
                                 Needs f16/bf16, 4 | b <= 16, 8 | in_f / b, 8 | r, y_out == NULL; else BLR_ERR_UNSUPPORTED */
  BLR_ALGO_STREAM_SPLIT = 4   /* the STREAM phases as separate launches (no grid barrier)   */
} blr_algo;

/* Monarch second factor: (l, s, r) for the right / right_ideal names, (l, r, s) for right_left
 * (reference models/wrappers.py:26-31).                                                      */
typedef enum { BLR_W2_SR = 0, BLR_W2_RS = 1 } blr_w2_layout;

/* Monarch output order: out[n, s*l + ll] (reference monarch_funcs.py:44) or the blocked
 * out[n, ll*S + s] of the right_ideal names (reference triton_funcs/monarch_kernels.py:1004). */
typedef enum { BLR_OUT_INTERLEAVED = 0, BLR_OUT_BLOCKED = 1 } blr_monarch_out;

/* Activation of the fused output stage (the *_fwd_ep entry points).  BLR_ACT_SILU_MUL is the gated unit of Llama's MLP over a
 * fused gate|up projection (reference configs/layers/llama7b.gate_up_proj.yaml:1-8: 4096 -> 22016 = gate | up): with
 * y = op(x) + bias and h = out_f / 2, out[m, c] = silu(y[m, c]) * y[m, c + h] - out then has h columns (ldo >= h). */
typedef enum { BLR_ACT_NONE = 0, BLR_ACT_GELU_TANH = 1, BLR_ACT_SILU = 2, BLR_ACT_SILU_MUL = 3 } blr_act;
typedef enum { BLR_OP_BLAST = 0, BLR_OP_MONARCH = 1, BLR_OP_LOW_RANK = 2, BLR_OP_DENSE = 3 } blr_op;

/* ---- workspaces ---------------------------------------------------------------------------
 * Every *_fwd entry point takes a caller-owned workspace of at least blr_*_workspace_bytes(...) bytes
 * for the same arguments.  For calls served by the streaming kernels (M <= 16 under BLR_ALGO_AUTO,
 * BLR_ALGO_STREAM, BLR_ALGO_STREAM_SPLIT) the workspace is more than scratch:
 *   - it must be ZERO-FILLED before its first use.  Its head (16 KiB of control words: barrier and
 *     check-in counters, the call epoch, the error word; then 32 KiB of arrival counters, 2 MiB of
 *     accumulation buffers and 16 MiB of tagged hand-over values) carries state from one call to the
 *     next: every value a workgroup hands to another is stored together with the epoch of its call,
 *     and a call recognises its own values by that tag;
 *   - nothing else may write to it between calls, and it must not be shared by calls that can
 *     overlap: one workspace per stream, calls on it stream-ordered;
 *   - the single-launch kernels wait for each other's values with every workgroup resident, so
 *     they expect the GPU to themselves while they run (a few microseconds); when another kernel
 *     occupies compute units at that moment a wait may run into its bound (about a second), the
 *     kernel then finishes with undefined results and records that in the workspace.  Such a
 *     give-up is reported by blr_workspace_status(), never by the call itself (which only enqueues).
 * Calls served by the tiled kernels (M > 16, BLR_ALGO_TILED) use the workspace as plain scratch.
 *
 * blr_workspace_status: SYNCHRONISES the stream, returns BLR_OK if no bounded wait gave up on this
 * workspace since the last query and BLR_ERR_TIMEOUT otherwise (the record is cleared; later calls
 * are valid again).  The reference's harness records a per-function FAIL in the same role
 * (reference layer.py:211-214, utils.py:8-13).  It must not be called while the stream is being
 * captured.
 * blr_set_spin_limit: polls after which a wait gives up, process-wide; 0 restores the default
 * (4,000,000, about a second).  Meant for tests of the give-up path.                          */
int blr_workspace_status(void* ws, size_t ws_bytes, void* stream);
void blr_set_spin_limit(unsigned polls);
/* The run-time switches of the library (no counterpart in the reference), all of them: the GEMM variant - BLR_GEMM_RING
 * (0..2), BLR_GEMM_RING_TILE (0, 256256, 256128, 256096, 128128), BLR_GEMM_RING_PER_CU (0..2), BLR_GEMM_RING_WAVES (4, 8),
 * BLR_GEMM_RING_BK (32, 64: k per operand stage), BLR_GEMM_SPLITK (0, 1) - and kernel families on / off - BLR_DECODE2, BLR_DECODE3, BLR_DECODE_ROWS, BLR_DENSE_SLAB,
 * BLR_DENSE_ROWS, BLR_BLAST_ONE, BLR_BLAST_YMIXW (0, 1), BLR_DECODE_PAIR, BLR_BLAST_MIXU (0..2); a family that is off hands its calls to the
 * next one that serves them.  Each starts from the environment variable of its name (read once; a value out of range is
 * ignored); unset != 0 returns it to "not set".  Returns BLR_ERR_BAD_ARG for an unknown name or a value out of range.  */
int blr_set_option(const char* name, int value, int unset);

const char* blr_last_error(void);
int blr_version(void);
/* Number of compute units of the current device (0 if no device). */
int blr_device_cus(void);

/* ---- BLAST --------------------------------------------------------------------------------
 * out[m, i*q + qq] = sum_r U_i[qq, r] * (sum_j S[i, j, r] * (sum_p x[m, j*p + pp] * V_j[pp, r]))
 * Replaces triton_blast_{partial,partial_grouped,partial_grouped_persistent,full}_{fp16,fp32}
 * (reference triton_funcs/blast_kernels.py:2614-2995; U (b,r,q), S (j,i,r)) and
 * triton_blast_bmm_{fp16,fp32} (:2998-3065; U (b,q,r), S (r,i,j)).  V is always (b, p, r).
 * y_out / z_out: optional (may be NULL) (b, M, r) buffers of dtype receiving the two
 * intermediates the *_fp32 names return.  They force the TILED algorithm.                    */
size_t blr_blast_workspace_bytes(int M, int in_f, int out_f, int b, int r, int dtype, int algo);
int blr_blast_fwd(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                  void* out, int64_t ldo, void* z_out, void* y_out,
                  int M, int in_f, int out_f, int b, int r,
                  int dtype, int u_layout, int s_layout, int algo,
                  void* ws, size_t ws_bytes, void* stream);

/* ---- BLAST with int8-valued intermediates ---------------------------------------------------
 * The arithmetic of the reference's blast_bmm_int8 kernels (triton_funcs/blast_sym_quant_kernels.py:
 * 92-112, 214-234, 340-360, launcher 558-580): Y = x_j V_j and Z = sum_j S Y are accumulated in fp32,
 * rounded to nearest even and saturated to [-128, 127]; out = Z_i U_i is stored in dtype.  Weights stay
 * in dtype (the reference kernels read them unquantized).  Same layouts and optional y_out / z_out as
 * blr_blast_fwd; the intermediates hold the int8 values exactly, in dtype.  Three launches at any M. */
size_t blr_blast_i8act_workspace_bytes(int M, int in_f, int out_f, int b, int r, int dtype);
int blr_blast_i8act_fwd(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                        void* out, int64_t ldo, void* z_out, void* y_out,
                        int M, int in_f, int out_f, int b, int r,
                        int dtype, int u_layout, int s_layout,
                        void* ws, size_t ws_bytes, void* stream);

/* ---- weight-quantized BLAST ---------------------------------------------------------------
 * Same product with U and V stored as symmetric int8 (bits = 8) or packed int4 (bits = 4) codes
 * and fp16 per-output-channel scales.  Both factors are stored (k, n)-ordered, the order in which
 * the kernels stream them: U codes (b, r, q[/2]) + u_scales (b, q); V codes (b, p, r[/2]) +
 * v_scales (b, r); S (r, i, j) of dtype.  Served behind the name triton_blast_bmm_int8_fp16
 * (reference triton_funcs/blast_sym_quant_kernels.py:558-580).  r % 8 == 0 and (out_f / b) % 8 == 0.
 * Up to 128 rows the kernels stream the codes and widen them in registers; larger M expands them to dtype in the
 * workspace first and runs the tiled kernels.  The quantizer and its code layout are this library's own: the reference
 * has no weight quantizer.                                                                                          */
size_t blr_blast_q_workspace_bytes(int M, int in_f, int out_f, int b, int r, int bits);
int blr_blast_q_fwd(const void* x, int64_t ldx,
                    const void* u_codes, const void* u_scales,
                    const void* v_codes, const void* v_scales, const void* S,
                    void* out, int64_t ldo,
                    int M, int in_f, int out_f, int b, int r,
                    int dtype, int bits, int algo,
                    void* ws, size_t ws_bytes, void* stream);

/* Symmetric per-channel quantizer producing the codes/scales consumed above.  w is viewed as
 * (outer, reduce, inner) contiguous; the max-abs runs over `reduce`.  scales: fp16 (outer, inner).
 * codes: int8 (outer, reduce, inner), or for bits = 4 two codes per byte along the flattened
 * last axis (low nibble = even index).  U (b, r, q): outer = b, reduce = r, inner = q; V (b, p, r):
 * outer = b, reduce = p, inner = r.  No reference counterpart (the reference has no weight
 * quantizer).                                                                                */
int blr_quantize_sym(const void* w, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                     int bits, void* codes, void* scales, void* stream);

/* ---- Monarch ------------------------------------------------------------------------------
 * w1 (b, in_f/b, rank) with pre-permuted columns (reference layer.py:221-224), w2 per
 * w2_layout.  Replaces triton_monarch_{right,right_ideal,right_left}_{fp16,fp32}
 * (reference triton_funcs/monarch_kernels.py:823-1099).  out1 (optional, may be NULL) receives
 * the permuted intermediate (b, M, rank) that the *_fp32 names return.                        */
size_t blr_monarch_workspace_bytes(int M, int in_f, int out_f, int b, int rank, int dtype, int algo);
int blr_monarch_fwd(const void* x, int64_t ldx, const void* w1, const void* w2,
                    void* out, int64_t ldo, void* out1,
                    int M, int in_f, int out_f, int b, int rank,
                    int dtype, int w2_layout, int out_order, int algo,
                    void* ws, size_t ws_bytes, void* stream);

/* ---- low rank -----------------------------------------------------------------------------
 * out = (x A) B with A (in_f, r), B (r, out_f).  Replaces triton_low_rank_{fp16,fp32}
 * (reference triton_funcs/low_rank_kernels.py:394-417).  z_out optional (M, r).              */
size_t blr_low_rank_workspace_bytes(int M, int in_f, int out_f, int r, int dtype, int algo);
int blr_low_rank_fwd(const void* x, int64_t ldx, const void* A, const void* B,
                     void* out, int64_t ldo, void* z_out,
                     int M, int in_f, int out_f, int r, int dtype, int algo,
                     void* ws, size_t ws_bytes, void* stream);

/* ---- dense --------------------------------------------------------------------------------
 * out = x W with W (in_f, out_f).  Replaces triton_dense_{fp16,fp32}
 * (reference triton_funcs/dense_kernels.py:360-381).                                         */
size_t blr_dense_workspace_bytes(int M, int in_f, int out_f, int dtype, int algo);
int blr_dense_fwd(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                  int M, int in_f, int out_f, int dtype, int algo,
                  void* ws, size_t ws_bytes, void* stream);

/* ---- bandwidth probe ----------------------------------------------------------------------
 * Streams `bytes` bytes from src with the load pattern of the streaming kernels and writes one
 * checksum word per workgroup to dst (dst needs 4 * blr_probe_dst_words() bytes).  Role of the
 * reference's *_load_store_* kernels (reference triton_funcs/dense_kernels.py:383-412,
 * low_rank_kernels.py:419-450): an empirical bandwidth ceiling for the decode kernels.        */
int blr_probe_dst_words(void);
int blr_stream_probe(const void* src, size_t bytes, void* dst, void* stream);
/* The whole memory pattern of a layer without its arithmetic, as the reference's load_store kernels have it
 * (reference triton_funcs/dense_kernels.py:150-227: load x, load w, store a zero y; low_rank_kernels.py:163-236
 * with two factors): every byte of x, w1 and (if w2_bytes > 0) w2 is loaded with the streaming pattern and
 * zeros are stored over all y_bytes of y.  All sizes are multiples of 16 and all pointers 16-byte aligned;
 * dst as for blr_stream_probe.                                                                          */
int blr_load_store_probe(const void* x, size_t x_bytes, const void* w1, size_t w1_bytes, const void* w2, size_t w2_bytes,
                         void* y, size_t y_bytes, void* dst, void* stream);

/* What the matrix cores sustain with nothing in their way (no counterpart in the reference; the role its device.py gives to a
 * spec-sheet number): one workgroup of eight waves per compute unit, each wave a chain of eight independent 32x32x16 fp16
 * products per iteration with the operands in registers.  random != 0: pseudo-random operands in [-2, 2) instead of ones (the
 * power drawn, and with it the clock, depends on the data); lds_reads = 6: every eight products come with the six 1 KiB
 * fragment reads from LDS that a 128 x 64 wave tile needs (0: none).  dst: at least 4 bytes of device memory.  Time the launch
 * with events; blr_mfma_probe_flops(iters) is the number of floating-point operations of one launch on the current device.   */
int blr_mfma_probe(int iters, int random, int lds_reads, void* dst, void* stream);
double blr_mfma_probe_flops(int iters);

/* ---- fused output stage ---------------------------------------------------------------------
 * out = act(op(x) + bias): what the callers do right after the operator - the bias add of the wrapper
 * modules (reference models/wrappers.py:176-177) and the activation that follows the first MLP linear
 * (GELU-tanh in DiT, reference DiT/models.py:111-112; SiLU in Llama).  bias: out_f values of dtype or NULL;
 * act: blr_act.  The other arguments are those of the entry point without the suffix.  Above 128 rows bias and
 * activation are applied while the last GEMM writes its tile out (to the result rounded to dtype, as the callers'
 * separate kernels would), so the M x out_f round trip of those kernels disappears; below, BLAST and Monarch apply them
 * in the output stage of their last few-row kernel (dense: at 17..128 rows with one slice), and what no kernel fuses is
 * finished by a small elementwise launch after the operator.                                                        */
int blr_blast_fwd_ep(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                     void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                     int dtype, int u_layout, int s_layout, int algo,
                     void* ws, size_t ws_bytes, void* stream, const void* bias, int act);
/* BLR_ACT_SILU_MUL (no reference kernel: it is the step Llama's MLP takes right after this path, act(gate) * up, on the
 * fused gate_up layer that reference configs/layers/llama7b.gate_up_proj.yaml:1-8 names): above 128 rows
 * of f16 / bf16, BLAST (even b), low rank and dense compute the tiles of the gate half and of the up half of an output position
 * in one work item of the last GEMM and write only the product, so the (M, out_f) intermediate never exists; everything else
 * (few rows, Monarch, fp32) computes the full-width result into the TAIL of the workspace and finishes with one elementwise
 * launch.  blr_ep_workspace_bytes: bytes to ADD to blr_*_workspace_bytes() for such a call (0 when the GEMM fuses it, and for
 * every other activation); op: blr_op; b: BLAST's number of blocks (ignored otherwise).                                      */
size_t blr_ep_workspace_bytes(int op, int M, int out_f, int b, int dtype, int act);
int blr_monarch_fwd_ep(const void* x, int64_t ldx, const void* w1, const void* w2,
                       void* out, int64_t ldo, int M, int in_f, int out_f, int b, int rank,
                       int dtype, int w2_layout, int out_order, int algo,
                       void* ws, size_t ws_bytes, void* stream, const void* bias, int act);
int blr_low_rank_fwd_ep(const void* x, int64_t ldx, const void* A, const void* B,
                        void* out, int64_t ldo, int M, int in_f, int out_f, int r, int dtype, int algo,
                        void* ws, size_t ws_bytes, void* stream, const void* bias, int act);
int blr_dense_fwd_ep(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                     int M, int in_f, int out_f, int dtype, int algo,
                     void* ws, size_t ws_bytes, void* stream, const void* bias, int act);

/* The same with a gate and a residual on top: out = resid + gate[m / gate_rows] * act(op(x) + bias), the adaLN-Zero update of a
 * DiT block (reference DiT/models.py:120-121: x = x + gate.unsqueeze(1) * attn(...) / mlp(...)), which the callers otherwise run as
 * separate elementwise kernels over the M x out_f result.  gate: (ceil(M / gate_rows), out_f) of dtype with row stride ld_gate, one
 * row per group of gate_rows consecutive rows (the tokens of one image), or NULL; resid: (M, out_f) of dtype with row stride
 * ld_resid, or NULL (it may be the same memory as out only if ldo == ld_resid: every element is read before it is written by the
 * same thread).  Fused into the write-out of the last GEMM at M > 16, an elementwise launch after the operator otherwise.   */
int blr_blast_fwd_ep2(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                      void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                      int dtype, int u_layout, int s_layout, int algo,
                      void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                      const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid);
int blr_monarch_fwd_ep2(const void* x, int64_t ldx, const void* w1, const void* w2,
                        void* out, int64_t ldo, int M, int in_f, int out_f, int b, int rank,
                        int dtype, int w2_layout, int out_order, int algo,
                        void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                        const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid);
int blr_low_rank_fwd_ep2(const void* x, int64_t ldx, const void* A, const void* B,
                         void* out, int64_t ldo, int M, int in_f, int out_f, int r, int dtype, int algo,
                         void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                         const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid);
int blr_dense_fwd_ep2(const void* x, int64_t ldx, const void* W, void* out, int64_t ldo,
                      int M, int in_f, int out_f, int dtype, int algo,
                      void* ws, size_t ws_bytes, void* stream, const void* bias, int act,
                      const void* gate, int gate_rows, int64_t ld_gate, const void* resid, int64_t ld_resid);

/* ---- BLAST forward that allocates nothing and takes no workspace -------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory or carry a workspace
 * around: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * arithmetic and arguments as blr_blast_fwd with BLR_ALGO_TILED (and the two-launch decode path at up
 * to four rows of f16 / bf16), without z_out / y_out / algo / ws: the intermediates live in a device
 * array built into the library, BLR_STATIC_SCRATCH_BYTES per GPU, held from the first call on that GPU
 * until the process ends.  A call whose intermediates do not fit (2 * b * M * r elements of dtype, each
 * half rounded up to 256 bytes) returns BLR_ERR_WORKSPACE; use blr_blast_fwd with a workspace then.
 * Calls no hipMalloc / hipFree and no allocating library routine.  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls ordered on one
 * stream are safe.  The kernels write all of the scratch they read, so nothing has to be cleared
 * between calls.  The first call on a device resolves the array's address (hipGetSymbolAddress); make
 * it outside a graph capture.                                                                       */
#define BLR_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
int blr_blast_fwd_static(const void* x, int64_t ldx, const void* U, const void* V, const void* S,
                         void* out, int64_t ldo, int M, int in_f, int out_f, int b, int r,
                         int dtype, int u_layout, int s_layout, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BLR_H */
