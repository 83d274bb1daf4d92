/*
 * dflash_mi355.h - C ABI of libdflash_mi355.so, the MI355X (gfx950) device side of
 * the dflash-mlx target-verify hot path.
 *
 * The reference reaches its device kernels through
 *   mx.fast.metal_kernel(name, input_names, output_names, source)(inputs=..., grid=...,
 *   threadgroup=..., output_shapes=..., output_dtypes=...)
 * (dflash_mlx/verify_qmm.py:120-125, 306-313, 323-330; dflash_mlx/kernels.py:393-406).
 * Each entry point below replaces one such launch site.  Conventions:
 *   - every pointer is caller-owned DEVICE memory unless named *_host;
 *   - kernels are enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *     default stream) and the call returns without waiting;
 *   - inputs are never written, outputs never alias inputs;
 *   - no entry point allocates device memory: scratch comes in as `workspace`;
 *   - return value 0 on success, a negative DFLASH_ERR_* otherwise (nothing is
 *     thrown across the boundary); dflash_last_error() describes the last failure
 *     on the calling thread.
 */
#ifndef DFLASH_MI355_H
#define DFLASH_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DFLASH_ABI_VERSION 18

enum {
  DFLASH_OK = 0,
  DFLASH_ERR_ARG = -1,       /* null pointer / unknown enum value            */
  DFLASH_ERR_SHAPE = -2,     /* shape the kernels do not cover               */
  DFLASH_ERR_WORKSPACE = -3, /* workspace missing or too small               */
  DFLASH_ERR_HIP = -4        /* a HIP runtime call failed                    */
};

enum { DFLASH_BF16 = 0, DFLASH_FP16 = 1, DFLASH_FP32 = 2 };

/* Shape dispatch of dflash_mlx/verify_qmm.py:19-22, 299-331. */
enum { DFLASH_QMM_MMA2BIG = 0, DFLASH_QMM_MMA2BIG_PIPE = 1 };

/*
 * Which device kernel serves a qmm call.  TILE: one workgroup per 32 output columns and
 * per K slice, K cut into k_parts slices for the pipe variant.  STREAM: persistent
 * workgroups that divide the weight matrix evenly and stream it through LDS; needs
 * group_size 64 and K % 512 == 0, and decides the K split itself (variant and k_parts
 * then only name the caller's dispatch decision).  AUTO: STREAM where it applies.
 */
enum { DFLASH_QMM_KERNEL_AUTO = 0, DFLASH_QMM_KERNEL_TILE = 1, DFLASH_QMM_KERNEL_STREAM = 2 };

int dflash_abi_version(void);
const char* dflash_last_error(void);

/*
 * Process-wide switches for tests and A/B measurements; no counterpart in the reference (whose
 * kernels have none).  They are plain integers read by the entry points named below, 0 (the
 * default) meaning "decide as documented"; nothing on a launch path reads the environment.
 *   DFLASH_OPT_GDN_STEP_BY_STEP  1: dflash_gdn_forward_tape{,_norm} keep the step-by-step kernel
 *                                where the block kernel would apply
 *   DFLASH_OPT_SDPA_SPLITS       n > 0: dflash_sdpa_q16 (and its workspace size) cut the keys into
 *                                n ranges (fewer if a range would fall below one tile)
 *   DFLASH_OPT_QMM_SPIN_LIMIT    n > 0: the streaming qmm kernel's workgroups that add partial tiles
 *                                give up after n polls instead of 2^22 (tests of that path: the
 *                                launch ends, the error word is set, results are unspecified)
 * dflash_set_option returns 0, or DFLASH_ERR_ARG for an unknown option or a negative value;
 * dflash_get_option returns the value, or DFLASH_ERR_ARG.
 */
enum {
  DFLASH_OPT_GDN_STEP_BY_STEP = 0,
  DFLASH_OPT_SDPA_SPLITS = 1,
  DFLASH_OPT_QMM_SPIN_LIMIT = 2,
  DFLASH_OPT_COUNT = 3
};
int dflash_set_option(int option, int value);
int dflash_get_option(int option);

/*
 * M=16 int4 affine quantized matmul, y[16,N] = x[16,K] . (scale*q + bias)^T.
 * Replaces the `verify_mma2big_*` launch (verify_qmm.py:323-330, variant
 * DFLASH_QMM_MMA2BIG, k_parts ignored) and the `verify_mma2big_pipe_*` launch plus
 * the host-side `partials.sum(axis=0).astype(T)` (verify_qmm.py:306-314, variant
 * DFLASH_QMM_MMA2BIG_PIPE: K is cut into k_parts contiguous slices whose fp32
 * partial products are summed in slice order and rounded once).
 *
 *   x        [16, K]            act_dtype (bf16 / fp16), row-major
 *   w_q      [N, K/8]           uint32, element k of row n = (w_q[n][k>>3] >> 4*(k&7)) & 15
 *   scales   [N, K/group_size]  sb_dtype (bf16 / fp16)
 *   biases   [N, K/group_size]  sb_dtype
 *   y        [16, N]            act_dtype
 *   workspace                   >= dflash_qmm_m16_workspace_bytes(...) bytes, 256-byte
 *                               aligned, ZERO-FILLED ONCE (all of it) by the caller before
 *                               its first use; every qmm kernel leaves it zero-filled, so
 *                               it can be reused by later calls on the same stream.
 *                               Calls that share a workspace must not overlap in time.
 * Requirements: group_size in {32,64,128}; N % 16 == 0; K % group_size == 0;
 * for the pipe variant K % (32*k_parts) == 0.  Results are deterministic
 * (bit-identical from run to run for identical inputs).
 *
 * The streaming kernel hands partial sums of row blocks that several workgroups share to one
 * of them through the workspace; that workgroup waits for the others' partial tiles (they
 * were dispatched before it, so they are running or done).  The wait is bounded: a workgroup
 * that gives up - which takes a device that keeps a workgroup of the launch from running for
 * several seconds - stores 0x80000000 | row block into the 32-bit word at byte offset
 * DFLASH_QMM_ERROR_OFFSET of the workspace, the launch ends normally, and y is then
 * undefined.  The word stays set until the caller zero-fills the workspace again, which it
 * must do before the next call; dflash_qmm_error() reads it.
 */
#define DFLASH_QMM_ERROR_OFFSET ((16384 - 64 + 1) * 4)
/* Copies the error word of a qmm workspace to *word_host (0: no wait has given up) after waiting
 * for the work enqueued on `stream`. */
int dflash_qmm_error(const void* workspace, uint32_t* word_host, void* stream);

size_t dflash_qmm_m16_workspace_bytes(int K, int N, int group_size, int variant, int k_parts,
                                      int kernel);

int dflash_qmm_m16(const void* x, const uint32_t* w_q, const void* scales, const void* biases,
                   void* y, void* workspace, size_t workspace_bytes, int K, int N, int group_size,
                   int act_dtype, int sb_dtype, int variant, int k_parts, int kernel, void* stream);

/*
 * dflash_qmm_m16 for callers that cannot allocate device memory: code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc.  No counterpart in the
 * reference (MLX allocates behind every array).  The workspace is an array inside the
 * library's own device image (DFLASH_QMM_STATIC_SCRATCH_BYTES, 8 MiB, held by
 * every GPU the library is used on until the process ends); the call allocates and frees
 * nothing.  Same operands, requirements, kernels and results (bit for bit) as dflash_qmm_m16.
 * A call whose workspace would not fit the array returns DFLASH_ERR_WORKSPACE: the dense
 * projections of the verify stacks need about 4 MiB; a pipe call served by the tile kernel
 * needs 64 KiB + k_parts * 64 * N bytes.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race, as they would on a
 * shared workspace.  Nothing but the product's own kernel is enqueued, also by the first call
 * on a GPU (the array reads zero when the library's image is loaded), so every call may be
 * made under stream capture.
 */
#define DFLASH_QMM_STATIC_SCRATCH_BYTES ((size_t)8 << 20)

int dflash_qmm_m16_static(const void* x, const uint32_t* w_q, const void* scales, const void* biases,
                          void* y, int K, int N, int group_size, int act_dtype, int sb_dtype,
                          int variant, int k_parts, int kernel, void* stream);

/*
 * Several qmm problems in one launch.  No counterpart in the reference, whose verify step
 * calls the kernel once per projection (dflash_mlx/verify_linear.py:103-143): a launch costs
 * more around its weight stream than inside it, so the projections of a layer are handed over
 * as one list and run back to back by one persistent grid - each divided among the workgroups
 * exactly as a dflash_qmm_m16 call of its own would be (streaming kernel), with results bit
 * for bit the same, the weights of the next problem already streaming while the current one
 * ends.
 *
 *   problems[i]: x [16, K], w_q [N, K/8], scales/biases [N, K/64], y [16, N] as for dflash_qmm_m16
 *               (layout DFLASH_QMM_LAYOUT_ROWS), or the packed images of dflash_qmm_m16_pack
 *               (DFLASH_QMM_LAYOUT_PACKED; same bits out, the loads of a wave then read consecutive memory).
 *               All problems of a launch share one layout.
 *   wait_for    -1, or the index j < i of the problem whose y is this problem's x (x == problems[j].y,
 *               K == its number of output columns): the x loads of problem i are held back until
 *               problem j's output has been stored; its weights stream regardless.
 *   epilogue    DFLASH_QMM_EPILOGUE_NONE, or DFLASH_QMM_EPILOGUE_SILU_MUL: w_q, scales, biases hold
 *               N/2 gate rows followed by N/2 up rows and y is [16, N/2],
 *                   g = round(gate), y = round(round(g * round(sigmoid(g))) * round(up))
 *               (round: to act_dtype), what `silu(gate_proj(x)) * up_proj(x)` of an MLP gives
 *               operator by operator with silu(x) = x * sigmoid(x).
 * Requirements: 1 <= count <= DFLASH_QMM_CHAIN_MAX; group_size 64; K % 1024 == 0; N % 16 == 0
 * (N % 128 == 0 with an epilogue); pointers 16-byte aligned; workspace of
 * dflash_qmm_m16_chain_workspace_bytes(...) bytes under the rules of dflash_qmm_m16 (zero-filled
 * once, reusable, shareable with the other qmm entry points on the same stream).
 * spin_limit bounds the wait for an earlier problem (polls of its counter; <= 0: a default of
 * several seconds).  A workgroup that gives up writes i + 1 into the 32-bit word at byte offset
 * DFLASH_QMM_CHAIN_ERROR_OFFSET of the workspace (it stays there until the caller clears it),
 * goes on with whatever x holds, and the launch ends normally: the outputs of problem i and of
 * what depends on it are then undefined.  The grid is one workgroup per compute unit, all of
 * which must be resident at once: the device must not be shared with other long-running kernels.
 * flags: 0, or DFLASH_QMM_CHAIN_JOINT_SPLIT for independent problems (every wait_for -1): the units
 * of all problems are laid end to end and divided among the workgroups as ONE range, so that
 * nearly every row block is computed by a single workgroup over all of K and only the row blocks
 * at the two ends of a workgroup's range go through partial tiles.  A row block's sum is then no
 * longer cut where a launch of its own would cut it: results equal dflash_qmm_m16's to within one
 * rounding of the output type instead of bit for bit, and are the same from run to run.  The
 * workspace size depends on the flag.
 */
#define DFLASH_QMM_CHAIN_MAX 16
#define DFLASH_QMM_CHAIN_ERROR_OFFSET DFLASH_QMM_ERROR_OFFSET
enum { DFLASH_QMM_EPILOGUE_NONE = 0, DFLASH_QMM_EPILOGUE_SILU_MUL = 1 };
enum { DFLASH_QMM_CHAIN_JOINT_SPLIT = 1 };
enum { DFLASH_QMM_LAYOUT_ROWS = 0, DFLASH_QMM_LAYOUT_PACKED = 1 };

typedef struct dflash_qmm_problem {
  const void* x;
  const uint32_t* w_q;
  const void* scales;
  const void* biases;
  void* y;
  int K, N;
  int wait_for;
  int epilogue;
  int layout; /* DFLASH_QMM_LAYOUT_ROWS, or DFLASH_QMM_LAYOUT_PACKED: w_q, scales, biases are the images
                 dflash_qmm_m16_pack wrote for this K and N - with the silu-mul epilogue those of
                 dflash_qmm_m16_pack_gate_up */
} dflash_qmm_problem;

size_t dflash_qmm_m16_chain_workspace_bytes(const dflash_qmm_problem* problems, int count, int group_size,
                                            int flags);

/*
 * Packed images of a gate/up matrix (N/2 gate rows followed by N/2 up rows) for a chained problem
 * with the silu-mul epilogue and DFLASH_QMM_LAYOUT_PACKED: row block rb holds the gate rows
 * 64 rb .. 64 rb + 63 and the up rows of the same output columns.  Sizes as
 * dflash_qmm_m16_packed_bytes(K, N, ...) gives them; group_size 64, K % 1024 == 0, N % 128 == 0.
 * dflash_qmm_m16_packed does not read these images.
 */
int dflash_qmm_m16_pack_gate_up(const uint32_t* w_q, const void* scales, const void* biases,
                                void* codes_out, void* scales_out, void* biases_out, int K, int N,
                                int group_size, void* stream);

int dflash_qmm_m16_chain(const dflash_qmm_problem* problems, int count, void* workspace,
                         size_t workspace_bytes, int group_size, int act_dtype, int sb_dtype,
                         int spin_limit, int flags, void* stream);

/*
 * The same product on weights stored in the order the streaming kernel consumes them.  No
 * counterpart in the reference (MLX keeps the row-major triple of dflash_mlx/verify_qmm.py:70-72
 * and its kernel gathers 4-byte words from it); a caller that may keep a second copy of a
 * linear's weights packs them once when the model is loaded (the place where
 * dflash_mlx/verify_linear.py:146-168 swaps the modules) and calls the packed form per step.
 * In the row-major form a 128-row block contributes 128 pieces of 128 bytes of codes and 256
 * pieces of 32 bytes of scales and biases per step along K, each piece a memory access of its
 * own; packed, every load instruction of a wave reads 1 KiB of consecutive memory.
 *
 *   codes   [ceil(N/128), K/256, 16 KiB]   scales, biases [ceil(N/128), K/1024, 4 KiB]
 *   (sizes from dflash_qmm_m16_packed_bytes; rows past N repeat row N-1)
 * Requirements: group_size 64, K % 1024 == 0, N % 16 == 0; all pointers 16-byte aligned; the
 * workspace of dflash_qmm_m16 (kernel = DFLASH_QMM_KERNEL_STREAM) with the same rules.
 * dflash_qmm_m16_packed returns bit for bit what dflash_qmm_m16 returns through the streaming
 * kernel for the unpacked operands.
 */
int dflash_qmm_m16_packed_bytes(int K, int N, int group_size, size_t* codes_bytes,
                                size_t* scales_bytes /* = biases bytes */);

int dflash_qmm_m16_pack(const uint32_t* w_q, const void* scales, const void* biases,
                        void* codes_out, void* scales_out, void* biases_out, int K, int N,
                        int group_size, void* stream);

int dflash_qmm_m16_packed(const void* x, const void* codes, const void* scales, const void* biases,
                          void* y, void* workspace, size_t workspace_bytes, int K, int N,
                          int group_size, int act_dtype, int sb_dtype, void* stream);

/*
 * Gathered per-expert M<=16-per-expert qmm for MoE layers: y[p,:] = x[p,:] . (s*q + b)^T of
 * expert expert_ids[p].  No counterpart in the reference tree: its MoE experts go through
 * mlx_lm's switch layers (third-party `mx.gather_qmm`), which `install_verify_linears`
 * (dflash_mlx/verify_linear.py:160) never swaps.  Rows of an expert are handled 16 at a time
 * as one MFMA tile; experts without rows cost one early-exit workgroup per column block.
 *
 *   x [P, K] act_dtype      expert_ids [P] int32 in [0, E)
 *   w_q [E, N, K/8] uint32  scales, biases [E, N, K/group_size] sb_dtype     y [P, N] act_dtype
 *   workspace               optional (may be NULL): >= dflash_qmm_m16_gather_workspace_bytes(...)
 *                           bytes, same rules as the workspace of dflash_qmm_m16 (zero-filled
 *                           once, reusable, shareable with it).  With a workspace, calls with
 *                           group_size 64, K % 512 == 0, P <= 256 and E <= 1024 are served by
 *                           the streaming kernel: the weights of the experts that have rows
 *                           are streamed through LDS by persistent workgroups, as for the
 *                           dense form.  Without one, or for other shapes, one workgroup per
 *                           (32 columns, expert) reads its weights directly.
 * Requirements: P <= 2048, group_size in {32,64,128}, N % 16 == 0, K % group_size == 0.
 * Rows whose expert id is outside [0, E) give zeros.  Deterministic.
 */
size_t dflash_qmm_m16_gather_workspace_bytes(int P, int K, int N, int E, int group_size);

int dflash_qmm_m16_gather(const void* x, const int32_t* expert_ids, const uint32_t* w_q,
                          const void* scales, const void* biases, void* y, void* workspace,
                          size_t workspace_bytes, int P, int K, int N, int E, int group_size,
                          int act_dtype, int sb_dtype, void* stream);

/*
 * GatedDeltaNet tape replay: for every slot s and value head hv apply the first
 * steps[s] recorded steps to the recurrent state,
 *     S[dv][dk] <- g_t * S[dv][dk] + k_t[dk] * delta_t[dv],   t = 0 .. steps[s]-1,
 * skipping steps whose mask byte is zero.  Replaces the `tape_replay{,_vec}{,_mask}`
 * launch of dflash_mlx/kernels.py:393-406 (kernel body :244-293).  The reference
 * slices the tape to the accepted length on the host (recurrent_rollback_cache.py:
 * 160-167); here the full tape is passed and the accepted length is an argument, read
 * from device memory when steps_dev is given so that it never has to visit the host.
 *
 *   tape      [slots, T, Hv, Dv]   tape_dtype (bf16 / fp16 / fp32)
 *   k         [slots, T, Hk, Dk]   k_dtype    (bf16 / fp16 / fp32), Hv % Hk == 0
 *   g         [slots, T, Hv] (g_per_dk = 0) or [slots, T, Hv, Dk] (g_per_dk = 1), g_dtype
 *   state_in  [slots, Hv, Dv, Dk]  state_dtype (fp32 / bf16 / fp16), Dk contiguous
 *   state_out same shape and dtype, must not alias state_in
 *   steps_dev [slots] int32 device array, or NULL to use steps_host for every slot;
 *             values are clamped to [0, T]
 *   mask      [slots, T] uint8 or NULL
 * exact_order != 0 forces the step-by-step evaluation order of the reference kernel
 * (always used for bf16/fp16 states, which are rounded after every step,
 * kernels.py:281-283); otherwise an fp32 state is updated through the algebraically
 * equal form  S = (prod g) S0 + sum_t (prod_{u>t} g_u) delta_t (x) k_t.
 * Requirements: Dk % 4 == 0, Dk <= 1024, T*(Dv + 2*Dk + 1)*4 bytes <= 64 KiB.
 */
int dflash_tape_replay(const void* tape, const void* k, const void* g, const void* state_in,
                       void* state_out, const int32_t* steps_dev, int steps_host,
                       const uint8_t* mask, int slots, int T, int Hk, int Hv, int Dk, int Dv,
                       int state_dtype, int tape_dtype, int k_dtype, int g_dtype, int g_per_dk,
                       int exact_order, void* stream);

/*
 * GatedDeltaNet forward over a block of T tokens that records the innovation tape - the
 * producer of what dflash_tape_replay consumes.  For every slot s and value head hv, with
 * hk = hv / (Hv / Hk), for t = 0 .. T-1 (steps whose mask byte is zero leave S alone and give
 * y_t = tape_t = 0):
 *     S <- g_t * S;  delta = (v_t - S k_t) * beta_t;  S <- S + delta (x) k_t;  y_t = S q_t;
 *     tape_t = delta;  S rounded through state_dtype.
 * Replaces the `gated_delta_tape{,_vec}{,_mask}` launch of dflash_mlx/kernels.py:207-224
 * (kernel body :29-106).
 *
 *   q, k      [slots, T, Hk, Dk]   in_dtype (bf16 / fp16 / fp32)
 *   v         [slots, T, Hv, Dv]   in_dtype
 *   g         [slots, T, Hv] (g_per_dk = 0) or [slots, T, Hv, Dk] (g_per_dk = 1), g_dtype
 *   beta      [slots, T, Hv]       beta_dtype
 *   state_in  [slots, Hv, Dv, Dk]  state_dtype, Dk contiguous; state_out same, no aliasing
 *   y         [slots, T, Hv, Dv]   in_dtype (output)
 *   tape      [slots, T, Hv, Dv]   fp32 (output)
 *   mask      [slots, T] uint8 or NULL
 * 128 x 128 heads take register-resident kernels: one gate per head with an fp32 state and
 * T <= 16 the block kernel on the fp32 matrix cores (closed form of the recurrence; the option
 * DFLASH_OPT_GDN_STEP_BY_STEP turns it off), the rest a step-by-step kernel
 * while T*(3*128 + (g_per_dk ? 128 : 1) + 2)*4 bytes fit 64 KiB of LDS; every other shape a
 * simple kernel that keeps S in state_out.
 */
int dflash_gdn_forward_tape(const void* q, const void* k, const void* v, const void* g,
                            const void* beta, const void* state_in, void* state_out, void* y,
                            float* tape, const uint8_t* mask, int slots, int T, int Hk, int Hv,
                            int Dk, int Dv, int in_dtype, int g_dtype, int beta_dtype,
                            int state_dtype, int g_per_dk, void* stream);

/*
 * The same forward with the layer's gated output norm applied to its result: what
 * dflash_mlx/runtime.py:441-448 computes with two calls (`gated_delta_kernel_with_tape`, then
 * `self.norm(out, z)`), in one launch where the block kernel applies (else the forward into
 * `out` followed by dflash_gdn_gated_norm in place).
 *     out = silu(z) * rms_norm(y, norm_weight, eps),  y the recurrence's output rounded to in_dtype
 *   z, out       [slots, T, Hv, Dv] in_dtype;  norm_weight [Dv] weight_dtype
 * Dv a multiple of 64 up to 256.  Everything else as for dflash_gdn_forward_tape.
 */
int dflash_gdn_forward_tape_norm(const void* q, const void* k, const void* v, const void* g,
                                 const void* beta, const void* state_in, void* state_out,
                                 const void* z, const void* norm_weight, void* out, float* tape,
                                 const uint8_t* mask, int slots, int T, int Hk, int Hv, int Dk, int Dv,
                                 int in_dtype, int g_dtype, int beta_dtype, int state_dtype,
                                 int weight_dtype, int g_per_dk, float eps, void* stream);

/*
 * GatedDeltaNet layer, everything between the input projections and the recurrence, in one
 * launch.  Replaces the array operators of dflash_mlx/runtime.py:381-407:
 *     qkv <- where(mask, qkv, 0);  conv_input = [conv_state | qkv] along the steps;
 *     conv_next = last conv_kernel-1 rows of conv_input;
 *     act = silu(depthwise_conv(conv_input));  q, k, v = split(act) into heads;
 *     q = Dk^-1 * rms_norm(q, eps);  k = Dk^-1/2 * rms_norm(k, eps);
 *     g = exp(-exp(A_log) * softplus(a + dt_bias));  beta = sigmoid(b).
 * Each of those operators rounds to `dtype` once (fp32 inside), a + dt_bias and the softplus
 * to the promoted type of `dtype` and `param_dtype`; g is fp32.
 *
 *   qkv         [B, S, C]  dtype, C = 2*Hk*Dk + Hv*Dv (q heads, k heads, v heads)
 *   conv_state  [B, conv_kernel-1, C] dtype, or NULL for zeros
 *   conv_w      [C, conv_kernel] dtype; tap j multiplies conv_input row s + j
 *   a, b        [B, S, Hv] dtype;  A_log, dt_bias [Hv] param_dtype;  mask [B, S] uint8 or NULL
 *   outputs: conv_next [B, conv_kernel-1, C], q, k [B, S, Hk, Dk], v [B, S, Hv, Dv], beta
 *   [B, S, Hv] in dtype; g [B, S, Hv] fp32.  Dk, Dv multiples of 64 up to 256; conv_kernel 2 to 4.
 */
int dflash_gdn_prepare(const void* qkv, const void* conv_state, const void* conv_w, const void* a,
                       const void* b, const void* A_log, const void* dt_bias, const uint8_t* mask,
                       void* conv_next, void* q, void* k, void* v, float* g, void* beta, int B,
                       int S, int Hk, int Hv, int Dk, int Dv, int conv_kernel, int dtype,
                       int param_dtype, float eps, void* stream);

/*
 * Gated output norm of a GatedDeltaNet layer: y = silu(z) * rms_norm(x, weight, eps) over rows of
 * length D (a multiple of 64 up to 256), x, z, y [rows, D] in dtype, weight [D] in weight_dtype.
 * Replaces `self.norm(out, z)` at dflash_mlx/runtime.py:448 (mlx-lm's Qwen3NextRMSNormGated).
 */
int dflash_gdn_gated_norm(const void* x, const void* z, const void* weight, void* y, long long rows,
                          int D, int dtype, int weight_dtype, float eps, void* stream);

/*
 * Exact attention of a verify block of 16 queries over a long KV cache.  Replaces the two
 * launches of dflash_mlx/kernels.py:735-761 (`batched_sdpa_2pass_partials{,_mask}` and
 * `batched_sdpa_2pass_reduce`): for batch b, query head hq, hk = hq / (Hq / Hk), query i < 16
 *     out[b, hq, i, :] = softmax_n(scale * q[b, hq, i, :] . k[b, hk, n, :] + mask[b, hq, i, n]) v[b, hk, n, :]
 * over the keys n <= N - 16 + i; with a mask, keys whose mask value is below the dtype's lowest
 * finite value are left out as well; a query without keys gives 0.
 *
 *   q, out  [B, Hq, 16, D]  dtype (bf16 / fp16), contiguous;  D = 128 or 256 (= value dim)
 *   k, v    element (b, h, n, d) at b * batch_stride + h * head_stride + n * seq_stride + d
 *           (strides in elements, multiples of 8): a KV cache is read in place
 *   mask    [B, Hq, 16, N] dtype, additive, or NULL
 *   workspace  dflash_sdpa_q16_workspace_bytes(B, Hq, Hk, N, D) bytes, 16-byte aligned, contents
 *           irrelevant (partial results of key ranges); may be NULL when that is 0
 * Hq a multiple of Hk, at most 8 query heads per key/value head; N >= 16.
 */
size_t dflash_sdpa_q16_workspace_bytes(int B, int Hq, int Hk, int N, int D);
int dflash_sdpa_q16(const void* q, const void* k, const void* v, const void* mask, void* out,
                    void* workspace, size_t workspace_bytes, int B, int Hq, int Hk, int N, int D,
                    long long k_batch_stride, long long k_head_stride, long long k_seq_stride,
                    long long v_batch_stride, long long v_head_stride, long long v_seq_stride,
                    float scale, int dtype, void* stream);

/*
 * Conv-window rebuild of a GatedDeltaNet layer after a partial acceptance: output
 * row j of a slot is row steps+j of concat([conv_prev, qkv], axis=rows).  Replaces the
 * array ops of dflash_mlx/recurrent_rollback_cache.py:129-146 (zeros stand in for a
 * missing conv_prev, :136-140).
 *
 *   conv_prev [slots, keep, C] or NULL    qkv [slots, T, C]    conv_out [slots, keep, C]
 *   elements of elem_bytes bytes, copied verbatim; steps as in dflash_tape_replay,
 *   clamped to [0, T]; keep = conv_kernel_size - 1.
 */
int dflash_conv_state_rebuild(const void* conv_prev, const void* qkv, void* conv_out,
                              const int32_t* steps_dev, int steps_host, int slots, int T, int keep,
                              int C, int elem_bytes, void* stream);

/*
 * Rollback of GatedDeltaNet layers in one launch: what dflash_tape_replay (no mask) and
 * dflash_conv_state_rebuild do, by one kernel whose trailing workgroups copy the conv-window
 * rows - what `RecurrentRollbackCache.rollback` (dflash_mlx/recurrent_rollback_cache.py:149-171)
 * does with its snapshot, its three tapes and the recorded qkv rows.  Operands, dtypes,
 * requirements and results (bit for bit) as for the two calls, with qkv [slots, T, C] holding
 * the same T rows per slot as the tapes; qkv NULL (or keep == 0) leaves the conv window out.
 * One launch and one trip through the caller's foreign-function interface per rollback.
 */
int dflash_rollback_layer(const void* tape, const void* k, const void* g, const void* state_in,
                          void* state_out, const void* conv_prev, const void* qkv, void* conv_out,
                          const int32_t* steps_dev, int steps_host, int slots, int T, int Hk,
                          int Hv, int Dk, int Dv, int state_dtype, int tape_dtype, int k_dtype,
                          int g_dtype, int g_per_dk, int exact_order, int keep, int C,
                          int qkv_elem_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DFLASH_MI355_H */
