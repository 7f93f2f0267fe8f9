/*
 * palimpsa_hip.h — C ABI of libpalimpsa_hip.so: the Palimpsa attention operator
 * on AMD MI355X (gfx950), hand-written HIP kernels.
 *
 * The library is the drop-in for the device side of the reference's operator
 * package palimpsa/ops/palimpsa/ (three Triton kernels and the Python that
 * launches them).  Plain pointers and sizes only; no torch types.
 *
 * Conventions
 *   - every buffer is owned by the caller, device-resident, densely packed:
 *       q,k [B,T,H,dk] (or [B,T,Hq,dk], see PalDims.n_qk_heads)  v,b,o,o_var [B,T,H,dv]  gt [B,T,H]  g,Ip [H]
 *       states [N,H,dv,dk] fp32 in (mu, I) form
 *     (layouts enforced by the reference through .contiguous():
 *      chunk_palimpsa_forgetting_scalar.py:14-20, and raw pointer arithmetic:
 *      fused_recurrent_palimpsa.py:60-66, :89-90).
 *   - varlen: B == 1, T == total tokens, cu_seqlens int32 [N+1] on the device.
 *   - kernels are enqueued on the caller's stream (a hipStream_t passed as
 *     void*); nothing synchronises, allocates or frees.
 *   - return value: 0 = ok; < 0 = argument error found before any HIP call
 *     (PAL_E_*); > 0 = a hipError_t from a launch.
 *   - row tensors and states are 16-byte aligned, the gate tensor gt 4-byte
 *     aligned whatever its element type (a bf16 gate is fetched as the aligned
 *     32-bit word that holds it); PAL_E_ALIGN otherwise.
 *   - dk and dv must be multiples of 16 in [16, 256]; callers with other sizes
 *     zero-pad (padding k,q,v,b with zeros leaves the valid outputs unchanged).
 */
#ifndef PALIMPSA_HIP_H
#define PALIMPSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PAL_ABI_VERSION 4

/* element types of tensors handed over the boundary */
#define PAL_DTYPE_F32 0
#define PAL_DTYPE_BF16 1

/* PalDims.flags */
#define PAL_FLAG_VARLEN 1u      /* cu_seqlens given (B must be 1)            */
#define PAL_FLAG_HAS_INIT 2u    /* init_mu / init_I given                    */
#define PAL_FLAG_STORE_FINAL 4u /* final_mu / final_I requested              */
#define PAL_FLAG_HAS_VAR 8u     /* o_var (fwd) / do_var (bwd) present        */
/* How the chunked entry points (pal_chunk_fwd, pal_gla_chunk_fwd, pal_gla_chunk_bwd) build the states at the start
 * of every tile; no counterpart in the reference, results agree to rounding.  Neither bit: chosen by shape.
 * Meant for tests and measurements. */
/* fp32 rows (dtype == PAL_DTYPE_F32) through the chunked entry points: by default every matrix product takes its
 * operands as sums of two bf16 numbers (three matrix instructions per product, fp32 accumulation), which keeps
 * outputs, states and gradients within 1e-4 (relative, max-norm) of the fp32 recurrence.  With this flag the fp32
 * rows are rounded to single bf16 / f16 operands like bf16 rows (errors of 1e-3 .. 1e-2, about twice as fast). */
#define PAL_FLAG_FP32_FAST 1024u
#define PAL_FLAG_STATES_TWO_KERNELS 256u /* per-tile contributions by all tiles in parallel, then a scan over
                                            the tiles (any shape and dtype)                                  */
#define PAL_FLAG_STATES_ONE_PASS 512u    /* one pass per (sequence, head) that keeps the running state in
                                            registers, wherever it applies (bf16 rows)                       */

/* pal_recurrent_fwd only (every other entry point answers PAL_E_STATE): init_mu and final_mu point to bf16 arrays of the
 * same shape.  A cache format for decode, where the state is all the traffic: 12 instead of 16 bytes per state entry
 * and step.  The precision state I stays fp32 (it accumulates small increments); mu is rounded to bf16 once per call,
 * an error of 2^-9 relative per call that decays with the forgetting factor.  No counterpart in the reference
 * (its states are fp32: fused_recurrent_palimpsa.py:84-96, :145-154). */
#define PAL_FLAG_STATE_MU_BF16 2048u

/* pal_chunk_fwd only: fill chunk_mu / chunk_I (and the final states when asked for) and leave the outputs alone; o and
 * o_var may be NULL.  For a backward whose forward did not keep the tile-start states: the token-serial entry point
 * hands long sequences to pal_chunk_bwd this way.  No counterpart in the reference. */
#define PAL_FLAG_STATES_ONLY 4096u

/* error codes (negative) */
#define PAL_OK 0
#define PAL_E_NULL -1        /* required pointer is NULL                      */
#define PAL_E_DIM -2         /* non-positive or out-of-range dimension        */
#define PAL_E_HEADDIM -3     /* dk or dv not a multiple of 16 in [16,256]     */
#define PAL_E_DTYPE -4       /* unsupported element type                      */
#define PAL_E_VARLEN_BATCH -5 /* cu_seqlens given with B != 1                 */
#define PAL_E_CU_SEQLENS -6  /* cu_seqlens not monotone / not starting at 0 / wrong total */
#define PAL_E_WORKSPACE -7   /* workspace missing or too small                */
#define PAL_E_CHUNK -8       /* unsupported chunk size                        */
#define PAL_E_STATE -9       /* init/final state flags and pointers disagree  */
#define PAL_E_CAPACITY -10   /* output table too small                        */
#define PAL_E_ALIGN -11      /* pointer not aligned (rows, states: 16 bytes; gt: 4 bytes) */
#define PAL_E_SCRATCH -12    /* the call needs more than the library's static scratch */

/* Bytes of device memory the library itself holds per GPU for pal_chunk_fwd_static. */
#define PAL_STATIC_SCRATCH_BYTES (64u << 20)

/* Tokens per chunk tile of the chunked kernels (the chunk size of the benchmark configurations). */
#define PAL_CHUNK 64

typedef struct PalDims {
  int32_t batch;        /* B (1 when varlen)                                  */
  int32_t seq_len;      /* T per batch row; total packed tokens when varlen   */
  int32_t n_seqs;       /* N: B, or number of documents when varlen           */
  int32_t n_heads;      /* H                                                  */
  int32_t dk;           /* key/query head dim                                 */
  int32_t dv;           /* value head dim                                     */
  int32_t total_chunks; /* chunk path: sum over sequences of ceil(len/PAL_CHUNK) */
  int32_t dtype;        /* PAL_DTYPE_* of q,k,v,b,o and of do,dq,dk,dv,db     */
  int32_t gate_dtype;   /* PAL_DTYPE_* of gt                                  */
  int32_t var_dtype;    /* PAL_DTYPE_* of o_var / do_var                      */
  uint32_t flags;       /* PAL_FLAG_*                                         */
  float scale;          /* output scale (reference default dk^-0.5)           */
  int32_t n_qk_heads;   /* heads of q, k, dq, dk: 0 or H = one per value head (the reference's layout); a divisor
                           Hq of H = q,k [B,T,Hq,dk], value head h reads q/k head h / (H / Hq) (what the layers
                           obtain by repeating heads, palimpsa/layers/meta_mamba2.py:281-282, palimpsa.py:266-267,
                           without materialising the repeat); dq, dk [B,T,Hq,dk] are summed over each group.
                           Every chunked and token-serial entry point takes it, pal_gla_* included (the
                           MetaMamba2 layer with its precision state off: meta_mamba2.py:281-282, :319-323). */
} PalDims;

/* Forward-side tensors.  Unused optional pointers are NULL. */
typedef struct PalFwdTensors {
  const void *q, *k, *v, *b;      /* dtype                                    */
  const void *gt;                 /* gate_dtype [B,T,H], 4-byte aligned       */
  const float *g, *Ip;            /* fp32 [H]                                 */
  void *o;                        /* dtype [B,T,H,dv]                         */
  void *o_var;                    /* var_dtype [B,T,H,dv] or NULL             */
  const float *init_mu, *init_I;  /* fp32 [N,H,dv,dk] or NULL                 */
  float *final_mu, *final_I;      /* fp32 [N,H,dv,dk] or NULL (may alias init_*) */
  const int32_t *cu_seqlens;      /* device int32 [N+1] or NULL               */
  const int32_t *chunk_table;     /* device int32 [total_chunks,4] (varlen chunk path) */
  const int32_t *chunk_offsets;   /* device int32 [N+1] (varlen chunk path)   */
  float *chunk_mu, *chunk_I;      /* fp32 [total_chunks,H,dv,dk]: state at the
                                     start of every chunk (chunk path)        */
} PalFwdTensors;

/* Backward-side tensors. */
typedef struct PalBwdTensors {
  const void *d_o;                /* dtype [B,T,H,dv]                         */
  const void *d_o_var;            /* var_dtype [B,T,H,dv] or NULL             */
  void *dq, *dk;                  /* dtype [B,T,H,dk]                         */
  void *dv, *db;                  /* dtype [B,T,H,dv]                         */
  float *dgt;                     /* fp32 [B,T,H]                             */
  float *dg, *dIp;                /* fp32 [H]                                 */
  float *d_init_mu, *d_init_I;    /* fp32 [N,H,dv,dk] or NULL                 */
} PalBwdTensors;

/* ------------------------------------------------------------------ queries */

/* Version of this interface (PAL_ABI_VERSION of the build). */
int pal_abi_version(void);

/* Text for a code returned by any pal_* function. */
const char *pal_strerror(int code);

/* Argument check shared by every entry point; no HIP call.  Replaces the
 * reference's ValueErrors for varlen misuse
 * (chunk_palimpsa_forgetting_scalar.py:629-630, fused_recurrent_palimpsa.py:273-277)
 * and extends them to everything a raw-pointer interface can get wrong. */
int pal_validate_dims(const PalDims *dims);

/* ------------------------------------------------------------- host helpers */

/* Chunk bookkeeping for packed variable-length batches, on the host.
 * Replaces fla.ops.utils.prepare_chunk_offsets / prepare_chunk_indices as used
 * at chunk_palimpsa_forgetting_scalar.py:633-641.
 *   cu_seqlens_host  int64 [n_seqs+1], cu[0] == 0, non-decreasing
 *   table_out        int32 [capacity,4] rows (seq, first_token, n_tokens, index_in_seq), or NULL to count only
 *   offsets_out      int32 [n_seqs+1] cumulative chunk counts, or NULL
 * Returns the total number of chunks (>= 0) or a PAL_E_* code. */
int pal_build_chunk_table(const int64_t *cu_seqlens_host, int32_t n_seqs, int32_t *table_out,
                          int32_t capacity, int32_t *offsets_out);

/* ---------------------------------------------------------- recurrent path */

/* Token-serial forward for any T >= 1 (T == 1 is single-step decode).
 * Replaces fused_palimpsa_recurrent_fwd and its kernel
 * (fused_recurrent_palimpsa.py:24-209), consuming bf16/fp32 rows directly
 * instead of the host-side fp32 casts of :226-236. */
int pal_recurrent_fwd(const PalDims *dims, const PalFwdTensors *t, void *stream);

/* Backward of pal_recurrent_fwd.  The reference has none
 * (fused_recurrent_palimpsa.py:250-253 raises NotImplementedError); gradients
 * follow the naive recurrence chunk_palimpsa_forgetting_scalar.py:669-725. */
size_t pal_recurrent_bwd_workspace_bytes(const PalDims *dims);
int pal_recurrent_bwd(const PalDims *dims, const PalFwdTensors *t, const PalBwdTensors *gr,
                      void *workspace, size_t workspace_bytes, void *stream);

/* -------------------------------------------------------------- chunked path */

/* Chunked forward.  Replaces ChunkPalimpsa.forward + chunk_palimpsa_fwd_kernel
 * (chunk_palimpsa_forgetting_scalar.py:66-218, :441-517).  Fills chunk_mu /
 * chunk_I (the reference's intermediate_mu_state / intermediate_I_state,
 * :187-188) for the backward.  The prefix products of the output kernel use f16
 * operands normalised per 64-token tile by three block exponents (of k, v and b),
 * so results do not depend on the magnitude of the rows; within a tile, entries
 * more than 2^26 below the largest of their tensor lose precision.  The state at
 * the start of a tile enters those products through the operands of the tile's
 * first token (as an f16 number: 11 bits, against the 8 of bf16 rows), and the
 * exponents of v and b are raised where that state is large against the rows.
 * cu_seqlens (varlen) must ascend from 0 to the token count; the kernels clamp
 * every sequence and tile to the token range, so a malformed array cannot make
 * them address memory beyond the tensors (results are then unspecified). */
int pal_chunk_fwd(const PalDims *dims, const PalFwdTensors *t, void *stream);

/* pal_chunk_fwd for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose wrapper allocates the
 * intermediate states with torch, chunk_palimpsa_forgetting_scalar.py:652-653).  Same tensors and results as
 * pal_chunk_fwd, except that the tile-start states are kept in a buffer of PAL_STATIC_SCRATCH_BYTES that the
 * library holds on every GPU it runs on (a static device array; nothing is allocated or freed by the call):
 *   - t->chunk_mu and t->chunk_I must be NULL (PAL_E_STATE otherwise); the states are not handed back, so no
 *     backward can follow this call;
 *   - total_chunks * n_heads * dv * dk * 8 bytes must fit: at most PAL_STATIC_SCRATCH_BYTES / 8 = 8 Mi state
 *     entries per call (e.g. H = 16, 64x64: 128 tiles = 8192 tokens; H = 16, 128x128: 32 tiles = 2048 tokens);
 *     PAL_E_SCRATCH otherwise.  Longer sequences are run in pieces through init_* / final_*;
 *   - all calls on one GPU share that GPU's buffer: calls that overlap in time on one GPU (different streams or
 *     threads) race on it.  Calls on one stream, or otherwise ordered, are fine; nothing has to be cleared between
 *     calls (every slot read by a call is written by that call first);
 *   - the first call on each GPU looks the buffer's address up (hipGetSymbolAddress); make it outside graph capture. */
int pal_chunk_fwd_static(const PalDims *dims, const PalFwdTensors *t, void *stream);

/* Chunked forward without the precision state (scalar-gated linear attention):
 *   S_t = exp(-gt_t g) S_{t-1} + v_t k_t^T,  o_t = scale S_t q_t.
 * Replaces the forward of fla.ops.simple_gla.chunk_simple_gla as the reference
 * layer calls it with metaplasticity off (palimpsa/layers/palimpsa.py:18,
 * :293-300; flash-linear-attention is a dependency of the reference, not part
 * of its tree).  Reads q, k, v, gt, g, [init_mu], cu_seqlens + chunk tables;
 * writes o, [final_mu] and, on this path, two buffers of total_chunks*H*dv*dk
 * entries: chunk_mu is fp32 scratch (free after the call; may be NULL when
 * pal_state_pass_applies(dims, 0) is 1), chunk_I receives the
 * tile-start states S in bf16 (2 bytes per entry; what the backward needs).
 * b, Ip, o_var, init_I, final_I are ignored; PAL_FLAG_HAS_VAR is rejected with
 * PAL_E_STATE.  init_mu / final_mu hold S as [N,H,dv,dk] fp32. */
int pal_gla_chunk_fwd(const PalDims *dims, const PalFwdTensors *t, void *stream);

/* Token-serial forward without the precision state (T >= 1; T == 1 is a decode
 * step).  Replaces fla.ops.simple_gla.fused_recurrent_simple_gla as called at
 * palimpsa/layers/palimpsa.py:298.  Same tensors as pal_gla_chunk_fwd without
 * the chunk arguments, except that init_mu / final_mu hold the state as
 * S [N,H,dk,dv] (the layout of the layer's cache on this path), so a step
 * streams the state once in and once out; they may be the same buffer. */
int pal_gla_recurrent_fwd(const PalDims *dims, const PalFwdTensors *t, void *stream);

/* Backward of pal_gla_chunk_fwd (replaces the backward of fla's chunk_simple_gla
 * for the same call site).  t as in the forward call, with chunk_I (bf16 tile
 * states) as that call left it, chunk_mu unused (may be NULL), t->o any valid
 * pointer (not read) and PAL_FLAG_STORE_FINAL clear.
 * Reads gr->d_o; writes gr->dq, dk, dv (dtype), gr->dgt (fp32 [B,T,H], gradient
 * of gt), gr->dg (fp32 [H], gradient of the per-head rate g) and, when not NULL,
 * gr->d_init_mu (fp32 [N,H,dv,dk]).  d_o_var, db, dIp, d_init_I are ignored.
 * Gradients flowing into the final state are not taken (as in pal_chunk_bwd). */
size_t pal_gla_chunk_bwd_workspace_bytes(const PalDims *dims);
int pal_gla_chunk_bwd(const PalDims *dims, const PalFwdTensors *t, const PalBwdTensors *gr,
                      void *workspace, size_t workspace_bytes, void *stream);

/* Chunked backward.  Replaces ChunkPalimpsa.backward + chunk_palimpsa_bwd_kernel
 * (chunk_palimpsa_forgetting_scalar.py:239-434, :519-620), including the host
 * side .sum(0) reductions of :609-613.  Needs chunk_mu / chunk_I as written by
 * pal_chunk_fwd on the same inputs.  Head dims: one kernel keeps a dk x dv
 * carry tile in LDS, so 4 dk (dv + 8) + 256 (max(dk, dv) + 4) + 32 dv + 288 must
 * not exceed 163840 (up to 128x192, 192x128, 256x64); PAL_E_HEADDIM otherwise.
 * fp32 rows without PAL_FLAG_FP32_FAST keep a second bf16 plane of that tile (8 dk (dv + 8) in the sum above)
 * and take head dims up to 128 (e.g. 96x96, 64x128, 128x64). */
size_t pal_chunk_bwd_workspace_bytes(const PalDims *dims);
int pal_chunk_bwd(const PalDims *dims, const PalFwdTensors *t, const PalBwdTensors *gr,
                  void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------ layer glue around the op */

/* The element-wise work the reference layer does either side of the operator
 * (palimpsa/layers/palimpsa.py:266-279 before, :337-343 after), each as one
 * kernel forward and one backward instead of a dozen framework kernels.
 * Rows are token-major; tokens = B*T (or the packed total). */
typedef struct PalGlueDims {
  int32_t tokens;
  int32_t n_heads;      /* H: heads of v/b/o (num_v_heads)                     */
  int32_t n_qk_heads;   /* heads of q_raw/k_raw; H is a multiple of it (:266-267) */
  int32_t dk, dv;       /* head dims, multiples of 8 in [8,256]                */
  int32_t dtype;        /* PAL_DTYPE_* of every row tensor                     */
  float eps;            /* prologue: clamp of the L2 norm (F.normalize, 1e-12);
                           epilogue: eps of the RMS norm                       */
  float dt_min, dt_max; /* prologue in the MetaMamba2 form (bs_raw NULL): bounds of the clamp on
                           softplus(dt_raw + dt_bias) (layers/meta_mamba2.py:284, time_step_limit) */
  int32_t norm_over_heads; /* epilogue: 0 = RMS norm over dv per head, gate after it (layers/palimpsa.py:337-343);
                           1 = gate first, RMS norm over all H*dv entries of a token with weight [H*dv] and
                           rstd [tokens] (layers/meta_mamba2.py:355-363); H*dv <= 4096 */
} PalGlueDims;

typedef struct PalPrologueTensors {
  const void *q_raw, *k_raw;       /* dtype [tokens,Hqk,dk] (after conv/SiLU)  */
  const void *x;                   /* dtype [tokens,H,dv]   (after conv/SiLU)  */
  const void *dt_raw, *bs_raw;     /* dtype [tokens,H]: dt_proj, bs_proj outputs */
  const void *b_raw;               /* dtype [tokens,H,dv]: b_proj output, or NULL */
  const float *dt_bias, *b_scale;  /* fp32 [H]                                 */
  void *q, *k;                     /* dtype [tokens,H,dk]                      */
  void *v, *b;                     /* dtype [tokens,H,dv]; b NULL iff b_raw NULL */
  float *gt;                       /* fp32 [tokens,H]                          */
} PalPrologueTensors;

typedef struct PalPrologueGrads {
  const void *dq, *dk;             /* dtype [tokens,H,dk]                      */
  const void *dv, *db;             /* dtype [tokens,H,dv]; db NULL iff b_raw NULL */
  const float *dgt;                /* fp32 [tokens,H]                          */
  void *dq_raw, *dk_raw;           /* dtype [tokens,Hqk,dk]                    */
  void *dx, *db_raw;               /* dtype [tokens,H,dv]                      */
  void *ddt_raw, *dbs_raw;         /* dtype [tokens,H]                         */
  float *ddt_bias, *db_scale;      /* fp32 [H]                                 */
} PalPrologueGrads;

/* Operator inputs from the projections (layers/palimpsa.py:266-279):
 *   q, k = l2norm(q_raw), l2norm(k_raw), heads repeated H/Hqk times
 *   bs = sigmoid(bs_raw) rounded to dtype;  v = x * bs
 *   b = sigmoid(b_raw) * softplus(b_scale) * bs          (when b_raw given)
 *   gt = softplus(dt_raw + dt_bias)                      (fp32)
 * With bs_raw NULL the call is the MetaMamba2 layer's (layers/meta_mamba2.py:283-299):
 *   gt = clamp(softplus(dt_raw + dt_bias), dt_min, dt_max);  v = x * gt;  b = sigmoid(b_raw) * softplus(b_scale) * gt
 * and q_raw, k_raw, q, k may all be NULL (that layer hands its B, C rows to the operator as they are,
 * shared heads through PalDims.n_qk_heads); dbs_raw, and with them dq, dk, dq_raw, dk_raw, are then unused. */
int pal_prologue_fwd(const PalGlueDims *dims, const PalPrologueTensors *t, void *stream);
/* Its backward.  workspace: pal_prologue_bwd_workspace_bytes(dims) bytes of
 * device memory for the per-head partial sums of ddt_bias / db_scale. */
size_t pal_prologue_bwd_workspace_bytes(const PalGlueDims *dims);
int pal_prologue_bwd(const PalGlueDims *dims, const PalPrologueTensors *t, const PalPrologueGrads *gr,
                     void *workspace, size_t workspace_bytes, void *stream);

typedef struct PalEpilogueTensors {
  const void *o;        /* dtype [tokens,H,dv]: operator output               */
  const void *x;        /* dtype [tokens,H,dv] or NULL (no residual, :337)    */
  const float *D;       /* fp32 [H] (with x)                                   */
  const void *gate;     /* dtype [tokens,H,dv]: g_proj output, or NULL (:340-343) */
  const float *weight;  /* fp32 [dv]: RMS norm weight                          */
  void *y;              /* dtype [tokens,H,dv]                                 */
  float *rstd;          /* fp32 [tokens,H]: 1/rms, kept for the backward       */
} PalEpilogueTensors;

typedef struct PalEpilogueGrads {
  const void *dy;       /* dtype [tokens,H,dv]                                 */
  void *d_o, *dx, *dgate; /* dtype [tokens,H,dv]; dx / dgate NULL iff x / gate NULL */
  float *dD;            /* fp32 [H] (with x)                                   */
  float *dweight;       /* fp32 [dv]                                           */
} PalEpilogueGrads;

/* y = rmsnorm(o + x*D) * weight * gate*sigmoid(gate)   (layers/palimpsa.py:337-343;
 * the gated norm is fla.modules.FusedRMSNormGated, a dependency outside the
 * reference tree: RMS norm over dv, then a swish gate).
 * With dims->norm_over_heads: y = rmsnorm_{H*dv}((o + x*D) * gate*sigmoid(gate)) * weight
 * (layers/meta_mamba2.py:355-363; fla.modules.layernorm_gated.RMSNormGated with norm_before_gate=False,
 * restated from its published behaviour), weight [H*dv], rstd [tokens]. */
int pal_epilogue_fwd(const PalGlueDims *dims, const PalEpilogueTensors *t, void *stream);
size_t pal_epilogue_bwd_workspace_bytes(const PalGlueDims *dims);
int pal_epilogue_bwd(const PalGlueDims *dims, const PalEpilogueTensors *t, const PalEpilogueGrads *gr,
                     void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------ shape queries */

/* 1 if the chunked entry points would build the tile-start states of this call (dims as handed to them,
 * including the PAL_FLAG_STATES_* bits) in one pass, 0 if with the two-kernel form.  With the one-pass form
 * pal_gla_chunk_fwd never touches its fp32 scratch (chunk_mu), which may then be NULL-sized by the caller. */
int pal_state_pass_applies(const PalDims *dims, int has_precision_state);

/* PAL_OK if pal_chunk_bwd serves this head-dim pair for rows of `dtype` under `flags` (PAL_FLAG_FP32_FAST is
 * the bit that matters), PAL_E_HEADDIM otherwise (see pal_chunk_bwd); lets a caller refuse in its forward what
 * its backward could not do. */
int pal_chunk_bwd_supported(int32_t dk, int32_t dv, int32_t dtype, uint32_t flags);

/* ------------------------------------------------------------ measurement */

/* Per-kernel timing aid; no counterpart in the reference.  While enabled, every
 * kernel launch of the library is bracketed by two HIP events on the launch
 * stream; pal_profile_read waits for the outstanding ones and returns the
 * accumulated time and launch count of one kernel.  This is the only state
 * of the library that calls share (launches of every thread are counted: the
 * backward entry points run on autograd's thread); the switch is atomic and
 * the counters are guarded by a mutex, so it is safe under concurrent callers.
 * Off by default; for benchmarks only. */
int pal_profile_enable(int on);               /* also resets the counters */
int pal_profile_kernel_count(void);
const char *pal_profile_kernel_name(int kernel_id);
int pal_profile_read(int kernel_id, double *total_ms, int64_t *launches);

#ifdef __cplusplus
}
#endif
#endif /* PALIMPSA_HIP_H */
