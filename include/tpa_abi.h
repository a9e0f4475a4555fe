/*
 * C ABI of libtpa_gfx950.so: Tensor Product Attention forward (prefill + decode), a
 * same-shape dense multi-head flash attention, and the backward pass of both, as hand-written
 * HIP kernels for gfx950.
 *
 * The reference has no native ABI.  Its operator boundary for this path is the Pallas call
 *   pl.pallas_call(_fwd_kernel, ...)(qa, qb, ka, kb, va, vb, q_segment_ids, kv_segment_ids) -> [o, l]
 * at tpa/tpa.py:492-543 (statics sm_scale, causal bound at tpa/tpa.py:493-500), reached from
 * tpa()/_tpa_fwd() (tpa/tpa.py:73-165) once per batch element through jax.vmap.  The entry
 * points below are what a jax.ffi / ctypes binding for that seam binds: plain pointers and
 * sizes, no torch or jax types.
 *
 * Common rules for every entry point
 *   - all pointers are device pointers owned by the caller; they must stay valid until the
 *     work enqueued on `stream` has completed;
 *   - calls only enqueue work on `stream` (a hipStream_t passed as void*; NULL = the null
 *     stream); they never synchronise, allocate or free device memory, throw or abort;
 *   - return 0 on success or a negative TPA_ERR_* code; an argument that fails validation is
 *     reported before anything is enqueued (TPA_ERR_LAUNCH, the runtime refusing one launch of a
 *     call that makes several, can leave the earlier ones enqueued);
 *   - re-entrant: may be called concurrently from several host threads.
 */
#ifndef TPA_ABI_H_
#define TPA_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPA_ABI_VERSION 9

/* element types of the factor / output arrays */
enum { TPA_DTYPE_F32 = 0, TPA_DTYPE_BF16 = 1 };

/* error codes (tpa_strerror gives text) */
enum {
  TPA_OK = 0,
  TPA_ERR_NULL = -1,        /* a required pointer is NULL */
  TPA_ERR_SHAPE = -2,       /* a dimension is <= 0 or exceeds what the kernels support */
  TPA_ERR_DTYPE = -3,       /* unknown dtype */
  TPA_ERR_ALIGN = -4,       /* pointer or stride not aligned as the selected kernel needs */
  TPA_ERR_WORKSPACE = -5,   /* workspace missing or too small */
  TPA_ERR_UNSUPPORTED = -6, /* the requested kernel cannot run this problem */
  TPA_ERR_LAUNCH = -7       /* the HIP runtime refused the launch */
};

/* which kernel family to use */
enum {
  TPA_KERNEL_AUTO = 0,    /* MFMA kernels when the problem qualifies, else the generic kernel */
  TPA_KERNEL_GENERIC = 1, /* any-shape fp32-math kernel */
  TPA_KERNEL_MFMA = 2     /* MFMA kernels only; TPA_ERR_UNSUPPORTED if the problem does not qualify */
};

/* values of the `causal` fields */
#define TPA_CAUSAL_NONE 0
#define TPA_CAUSAL_TOP_LEFT 1     /* the reference's mask (tpa/tpa.py:377-379) */
#define TPA_CAUSAL_BOTTOM_RIGHT 2 /* an addition: see TpaFwdArgs.causal_offset */

/* TpaFwdArgs.nomat */
#define TPA_NOMAT_OFF 0
#define TPA_NOMAT_SPLIT_KEYS 1
#define TPA_NOMAT_RANK_PAIRS 2

/*
 * One factor array: A factors a[b, l, r, h] or B factors b[b, l, r, d].  The innermost
 * dimension is contiguous; the other three have ELEMENT strides, so both the split arrays
 * qa[lq, rq, h] / qb[lq, rq, dk] of tpa/tpa.py:246-251 and the concatenated q[b, lq, rq, h+dk]
 * of tpa/tpa.py:75-77 (A = base, B = base + h, rank stride h+dk) are read in place.
 */
typedef struct TpaFactor {
  const void* ptr;
  int64_t stride_b; /* elements between batch entries */
  int64_t stride_l; /* elements between tokens */
  int64_t stride_r; /* elements between ranks */
} TpaFactor;

/*
 * tpa_fwd / tpa_decode arguments.  Replaces the operand list and statics of the pallas_call at
 * tpa/tpa.py:492-543.  Semantics (tpa/tpa.py:245-443):
 *   Q = (1/rq) sum_r qa_r (x) qb_r, K, V likewise with 1/rk           (tpa/tpa.py:317,364,417)
 *   x = sm_scale * Q K^T                                              (tpa/tpa.py:365-367)
 *   masked (-inf) where segment ids differ or, if causal, key index > query index
 *                                                                      (tpa/tpa.py:369-386)
 *   lse = logsumexp_k x ; o = softmax_k(x) V                          (tpa/tpa.py:389-424)
 *   rows with every key masked: o = NaN, lse = -inf                   (tpa/tpa.py:437-439)
 */
typedef struct TpaFwdArgs {
  TpaFactor qa; /* [B, lq, rq, H]  */
  TpaFactor qb; /* [B, lq, rq, dk] */
  TpaFactor ka; /* [B, lk, rk, H]  */
  TpaFactor kb; /* [B, lk, rk, dk] */
  TpaFactor va; /* [B, lk, rk, H]  */
  TpaFactor vb; /* [B, lk, rk, dv] */
  const int32_t* q_segment_ids;  /* [B, lq] contiguous, or NULL (then kv_segment_ids must be NULL) */
  const int32_t* kv_segment_ids; /* [B, lk] contiguous, or NULL */
  void* o;      /* [B, lq, H, dv] contiguous, element type = dtype (tpa/tpa.py:529) */
  float* lse;   /* [B, H, lq] contiguous fp32 natural-log logsumexp, or NULL to skip it.
                   The reference's l[lq, h] (tpa/tpa.py:530) is the transpose of one batch entry. */
  int32_t B, lq, lk, H, dk, dv, rq, rk;
  int32_t dtype;  /* TPA_DTYPE_*: element type of the six factor arrays and of o */
  float sm_scale; /* multiplies the logits after the dot product (tpa/tpa.py:367) */
  int32_t causal; /* TPA_CAUSAL_*: 0 none; 1 key index <= query index, top-left aligned (tpa/tpa.py:377-379);
                     2 the last query aligned with the last key of each batch entry */
  int32_t kernel; /* TPA_KERNEL_* */
  void* workspace;        /* required by tpa_decode (split partials); optional for tpa_fwd (tpa_fwd_workspace_bytes) */
  size_t workspace_bytes; /* size of workspace */
  int32_t num_splits;     /* tpa_decode only: 0 = choose; otherwise the number of key ranges */
  const int32_t* kv_lengths; /* [B] or NULL: batch entry b attends to its first min(kv_lengths[b], lk) keys only,
                                the rest of its k / v arrays is not read (sequences of different lengths in one
                                padded cache; 0 = no key: o = NaN, lse = -inf).  No counterpart in the reference,
                                which would express this with segment ids (tpa/tpa.py:369-375). */
  /* Paged cache (tpa_decode's split-key kernel only; TPA_ERR_UNSUPPORTED elsewhere).  With page_table != NULL
     ka / kb / va / vb are page pools [page, token_in_page, rank, x] (stride_b = elements between pages) and token
     t of batch entry b lives in page page_table[b * pages_per_seq + t / page_size] at slot t % page_size.
     page_size * rk must be a multiple of 32 and pages_per_seq * page_size >= lk.  No counterpart in the reference. */
  const int32_t* page_table; /* [B, pages_per_seq] or NULL */
  int32_t page_size;         /* tokens per page */
  int32_t pages_per_seq;     /* entries per row of page_table */
  /* With causal == TPA_CAUSAL_BOTTOM_RIGHT the offset below counts from (keys of the batch entry - lq), the keys of
     an entry being min(kv_lengths[b], lk): lq freshly appended tokens per sequence of a ragged batch, each masked to
     its predecessors, need no offset at all.
     With causal != 0: key index <= query index + causal_offset.  0 is the reference's top-left alignment
     (tpa/tpa.py:377-379); lk - lq aligns the last query with the last key (a chunk of new tokens over a
     cache); a sequence shard passes the distance between its first query and the first key of the key shard
     it meets (tpa/ring_tpa.py:73-79 calls the block function with local indices only).  Rows that see no key
     end as NaN / -inf like any other empty row.  tpa_fwd and tpa_decode; ignored when causal == 0. */
  int32_t causal_offset;
  /* tpa_fwd only; stands where the reference kernel has its static `nomat` (tpa/tpa.py:250): never form K or V.
     The result is the same function of the inputs as with nomat == 0 (tpa/tpa_test.py:122-190 runs one grid over
     both), in another order of operations.  Never chosen by the library itself.
     TPA_NOMAT_SPLIT_KEYS (1): the split-key kernels of tpa_decode over windows of at most 64 query rows (two
       launches per window).  Per head they form Qm[h] = (1/rq) sum_r qa_r[h] qb_r once, the logits are
       (sm_scale / rk) sum_s ka_s[h] (kb_s . Qm[h]) and o = (1/rk) sum_s (sum_k p_k va_s[k, h]) vb_s
       (tpa/tpa.py:398-413), so every head shares one pass over the kb / vb rows; Q is still formed per head.
       Needs args.workspace >= tpa_fwd_nomat_workspace_bytes(...) (else TPA_ERR_WORKSPACE) and the shapes those
       kernels take (dk == dv in {64, 128}, rk a power of two <= 32, no segment ids; bf16 also H % 8 == 0 and
       16-byte aligned factors).  The faster of the two; it is what tpa_decode is.
     TPA_NOMAT_RANK_PAIRS (2): the reference's own arithmetic (tpa/tpa.py:333-359): a table bb = kb_s . qb_r per
       rank pair and block of keys that the heads of a workgroup share, combined per head with qa_r ka_s; neither
       Q nor K nor V is formed.  One launch, no workspace; bf16, dk == dv in {64, 128}, rq in {1, 6},
       rk in {1, 2, 4}, no segment ids, 16-byte aligned B factors and output.
     Any other problem runs the generic kernel (TPA_ERR_UNSUPPORTED with kernel == TPA_KERNEL_MFMA). */
  int32_t nomat;
} TpaFwdArgs;

/*
 * mha_fwd arguments: dense attention with the layouts of mha() at tpa/mha.py:11-17,
 *   q[B, lq, H, dk]  k[B, lk, H, dk]  v[B, lk, H, dv]  ->  o[B, lq, H, dv],
 * x = sm_scale * q k^T (+ bias[b, lq, lk] broadcast over heads, tpa/mha.py:31-34), softmax, p v.
 * `causal` is an addition: the reference expresses causality as a dense -inf bias
 * (tpa/tpa_test.py:52-54).  A dense bias is honoured by the generic kernel only.
 */
typedef struct MhaFwdArgs {
  const void* q; /* token stride = H*dk, batch stride = lq*H*dk (contiguous) */
  const void* k;
  const void* v;
  const float* bias; /* [B, lq, lk] fp32 additive, or NULL */
  void* o;
  float* lse; /* [B, H, lq] fp32 or NULL */
  int32_t B, lq, lk, H, dk, dv;
  int32_t dtype;
  float sm_scale;
  int32_t causal;
  int32_t kernel;
  void* workspace;        /* used when lq is small (split over keys), else ignored */
  size_t workspace_bytes;
  int32_t num_splits;
} MhaFwdArgs;

/*
 * One gradient array, fp32 whatever the element type of the inputs is: same indexing as the
 * TpaFactor it is the gradient of (innermost dimension contiguous, ELEMENT strides), so the
 * concatenated dq[b, lq, rq, h+dk] that _tpa_bwd returns (tpa/tpa.py:960-962) is written in place
 * (A part = base, B part = base + h, rank stride h+dk).
 */
typedef struct TpaGrad {
  float* ptr;
  int64_t stride_b;
  int64_t stride_l;
  int64_t stride_r;
} TpaGrad;

/*
 * tpa_bwd arguments.  Replaces the operand list of pl.pallas_call(_bwd_kernel, ..., name="tpa_bwd")
 * at tpa/tpa.py:872-958 together with _precompute_delta (tpa/tpa.py:965-995), for all batch
 * entries at once (the reference vmaps _bwd, tpa/tpa.py:191-213).  With x, p as in the forward pass:
 *   delta = sum_d o * do (NaN products skipped)                        (tpa/tpa.py:979)
 *   p = exp(x - lse), 0 where masked or where the row has no visible key  (tpa/tpa.py:675-676)
 *   dV = p^T do ; dp = do V^T ; ds = sm_scale * p * (dp - delta)       (tpa/tpa.py:765-773)
 *   dK = ds^T Q ; dQ = ds K                                            (tpa/tpa.py:775-781)
 *   da_r = (1/R) dX . b_r ; db_r = (1/R) a_r . dX  for X in {Q, K, V}  (tpa/tpa.py:767-768,776-777,782-783)
 * Every element of the six gradient arrays is written (no accumulation into their old contents).
 */
typedef struct TpaBwdArgs {
  TpaFactor qa, qb, ka, kb, va, vb;  /* the forward inputs, as in TpaFwdArgs */
  const int32_t* q_segment_ids;      /* [B, lq] or NULL */
  const int32_t* kv_segment_ids;     /* [B, lk] or NULL */
  const void* o;     /* [B, lq, H, dv] forward output, element type = dtype */
  const float* lse;  /* [B, H, lq] forward logsumexp (fp32) */
  const void* d_o;   /* [B, lq, H, dv] gradient of the loss with respect to o, element type = dtype */
  TpaGrad dqa, dqb, dka, dkb, dva, dvb; /* outputs, fp32 */
  int32_t B, lq, lk, H, dk, dv, rq, rk;
  int32_t dtype;
  float sm_scale;
  int32_t causal;
  int32_t kernel;         /* TPA_KERNEL_*: the MFMA kernels take bf16 or fp32 with dk == dv in {64, 128}; d_o must be 16-byte aligned */
  void* workspace;        /* required: at least tpa_bwd_workspace_bytes(...) bytes, 256-byte aligned */
  size_t workspace_bytes;
  int32_t causal_offset;  /* as in TpaFwdArgs: the value the forward call was made with */
} TpaBwdArgs;

/*
 * mha_bwd arguments: gradients of dense attention, _mha_bwd at tpa/mha.py:40-65, recomputing p
 * from (q, k, lse) instead of keeping the [b, h, lq, lk] matrix the reference saves
 * (tpa/mha.py:37).  dq, dk_out, dv_out are fp32, contiguous, with the shapes of q, k, v.
 */
typedef struct MhaBwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const float* bias; /* [B, lq, lk] fp32 additive or NULL; no gradient is produced for it (tpa/mha.py:64) */
  const void* o;
  const float* lse;
  const void* d_o;
  float* dq;
  float* dk_out;
  float* dv_out;
  int32_t B, lq, lk, H, dk, dv;
  int32_t dtype;
  float sm_scale;
  int32_t causal;
  int32_t kernel;
  void* workspace;        /* required: at least mha_bwd_workspace_bytes(...) bytes, 256-byte aligned */
  size_t workspace_bytes;
} MhaBwdArgs;

/*
 * tpa_cache_append arguments: the producer step of a TPA layer for n new tokens per sequence.  No
 * counterpart in the reference, which takes the factors as given (tpa/tpa.py:74-77); this is the
 * step that makes them (arXiv 2501.06425, section 3: the factors are linear in the hidden state and
 * rotary position embedding is applied to the B factors of Q and K) and appends the K / V factors
 * to the cache that tpa_decode and tpa_fwd read:
 *   y[b, i, :] = W x[b, i, :]                      W[n_out, d_model] row-major (out, in), columns of y in
 *                                                  the order qa[rq*H] qb[rq*D] ka[rk*H] kb[rk*D] va[rk*H] vb[rk*D]
 *   qb, kb: each rank row rotated pairwise, (y[2j], y[2j+1]) by the angle of position pos and
 *           frequency j:  y'[2j] = y[2j] c - y[2j+1] s,  y'[2j+1] = y[2j+1] c + y[2j] s,
 *           c = rope_cos[pos, j], s = rope_sin[pos, j]
 *   pos = positions[b, i] if given, else kv_lengths[b] + i (0 + i without kv_lengths)
 *   qa, qb are written to the q arrays at token i; ka, kb, va, vb at token kv_lengths[b] + i of batch
 *   entry b's cache (contiguous, or paged exactly as in TpaFwdArgs).  Tokens that would land at or
 *   beyond cache_len are dropped.  new_kv_lengths[b] = min(kv_lengths[b] + n, cache_len) if given.
 * The 1/R of the reconstruction is not applied here (tpa_fwd / tpa_decode apply it).
 */
typedef struct TpaAppendArgs {
  const void* x;          /* [B, n, d_model] contiguous, element type = dtype */
  const void* w;          /* [rq*(H+D) + 2*rk*(H+D), d_model] contiguous, element type = dtype */
  const float* rope_cos;  /* [rope_len, D/2] fp32 */
  const float* rope_sin;  /* [rope_len, D/2] fp32 */
  const int32_t* positions;   /* [B, n] or NULL */
  const int32_t* kv_lengths;  /* [B] tokens already in each cache, or NULL (= 0) */
  int32_t* new_kv_lengths;    /* [B] or NULL; must not alias kv_lengths */
  TpaFactor qa, qb;           /* outputs [B, n, rq, H], [B, n, rq, D] (ptr is written through) */
  TpaFactor ka, kb, va, vb;   /* the cache, [B, cache_len, rk, H|D] or page pools (ptr is written through) */
  const int32_t* page_table;  /* as in TpaFwdArgs, or NULL */
  int32_t page_size, pages_per_seq;
  int32_t B, n, d_model, H, D, rq, rk;  /* H % 8 == 0 and D % 8 == 0 for every kernel of this call (outputs are written
                                           in 16-byte chunks of 8 columns that must not straddle two arrays), else TPA_ERR_SHAPE */
  int32_t cache_len;          /* token capacity of one sequence (paged: pages_per_seq * page_size) */
  int32_t rope_len;           /* rows of the rotary tables: positions are clamped to rope_len - 1 */
  int32_t dtype;              /* TPA_DTYPE_*: element type of x, w, the q outputs and the cache */
  int32_t kernel;             /* TPA_KERNEL_*: the MFMA kernel takes bf16 with d_model % 64 == 0, H % 8 == 0, D % 8 == 0 */
  void* workspace;            /* optional (NULL: none), 16-byte aligned: see tpa_cache_append_workspace_bytes */
  size_t workspace_bytes;
} TpaAppendArgs;

/*
 * Projections to the rank factors, rotary embedding and append to the factored cache (see
 * TpaAppendArgs).  Enqueues one kernel on `stream` and needs no workspace; a decode step (at most 64
 * new tokens in all) that brings tpa_cache_append_workspace_bytes(...) bytes runs as two kernels that
 * split the contraction over more workgroups (fp32 partial sums in the workspace, same results up to
 * the order of the fp32 additions).
 */
int tpa_cache_append(const TpaAppendArgs* args, void* stream);

/* Bytes of optional workspace with which tpa_cache_append can split the contraction of a decode step
   over workgroups, 0 if it would not use one (more than 64 new tokens, dtype or d_model not eligible). */
size_t tpa_cache_append_workspace_bytes(int32_t B, int32_t n, int32_t d_model, int32_t H, int32_t D, int32_t rq, int32_t rk, int32_t dtype);

/* ABI version of the loaded library (TPA_ABI_VERSION it was built with). */
int tpa_abi_version(void);

/* Text for an error code returned by the functions below. */
const char* tpa_strerror(int code);

/*
 * Forward pass for any lq (prefill).  Replaces pl.pallas_call(..., name="tpa_fwd") at
 * tpa/tpa.py:492-543 for all batch entries at once (the reference vmaps it, tpa/tpa.py:144-163).
 * If `workspace` holds at least tpa_decode_workspace_bytes(...) bytes and the problem is a
 * decode (lq <= 16, lk >= 1024, no segment ids) that tpa_decode's kernel takes, the call is served by
 * it; if `workspace` holds tpa_fwd_workspace_bytes(...) bytes and the problem is long enough for it to
 * pay (rank 2: 2048 query rows and more; other ranks: more than 256), dense bf16 Q (times
 * sm_scale * log2 e), K and V are reconstructed into it once and the prefill kernel runs its loop over
 * dense tiles.  Without a workspace the same problems run on the fused prefill kernel, which rebuilds
 * K / V tiles from the rank factors inside its loop.  The two routes round at the same points (Q, K, V,
 * the probabilities and the output to bf16 once each) but are not bit-identical.
 */
int tpa_fwd(const TpaFwdArgs* args, void* stream);

/*
 * Bytes of optional workspace (256-byte aligned) with which tpa_fwd can pick a faster kernel for
 * this problem, 0 if none would be used: the split partials of the decode kernel (lq <= 16 over
 * a long cache), or room for dense bf16 K, V [B, lk, H, D] and Q [B, lq, H, D] (the reference
 * reconstructs them per pair of blocks, tpa/tpa.py:317,364,417).
 */
size_t tpa_fwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t rq, int32_t rk);

/*
 * Bytes of workspace (256-byte aligned) tpa_fwd needs with args.nomat != 0 for the split-key kernels to serve
 * the problem, 0 if its head sizes or rank are not theirs (then the generic kernel runs and needs none).  The
 * same workspace serves every window of query rows in turn.
 */
size_t tpa_fwd_nomat_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t rq, int32_t rk);

/*
 * Forward pass for few query tokens over a long factored cache (the reference reaches this as
 * the same call with lq = 1: block_q = min(128, lq), tpa/tpa.py:485).  Keys are split into
 * ranges whose partial (o, lse) are merged with the rule of _lse_accum (tpa/tpa.py:228-242).
 * Needs `workspace` of at least tpa_decode_workspace_bytes(...) bytes.  The causal mask is a
 * key count per query row (row i reads its first i + causal_offset + 1 keys); segment ids are
 * not supported (must be NULL): TPA_ERR_UNSUPPORTED otherwise.
 */
int tpa_decode(const TpaFwdArgs* args, void* stream);

/*
 * tpa_decode without a caller workspace.  No counterpart in the reference: it exists for callers
 * that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  Same arguments, kernels and results as tpa_decode, but args->workspace
 * and args->workspace_bytes are ignored: the split partials go to a fixed device array of
 * TPA_DECODE_NOALLOC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process
 * ends.  Problems whose partials (tpa_decode_workspace_bytes) exceed that size return
 * TPA_ERR_WORKSPACE; problems the split-key kernels do not take return TPA_ERR_UNSUPPORTED (there is
 * no fallback to the vector-ALU kernel here).  The call allocates and frees nothing; the first call
 * on a device looks up the array's device address (make that call outside a graph capture).  All
 * calls on one GPU share the array: calls that overlap in time on one GPU (different streams, or
 * several host threads) race on it and must be serialised by the caller.
 */
#define TPA_DECODE_NOALLOC_SCRATCH_BYTES (8u << 20)
int tpa_decode_noalloc(const TpaFwdArgs* args, void* stream);

/* Bytes of workspace tpa_decode needs for this problem (num_splits = 0: the default choice). */
size_t tpa_decode_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dv, int32_t num_splits);

/* Number of key ranges tpa_decode_workspace_bytes sizes the workspace for when num_splits == 0: what
   the bf16 kernel uses, and an upper bound on what the fp32 kernel uses (it serves one query row per
   workgroup and so asks for at most as many ranges). */
int32_t tpa_decode_default_splits(int32_t B, int32_t lq, int32_t lk, int32_t H);

/* Dense attention forward with the layouts of tpa/mha.py:11-17 (see MhaFwdArgs). */
int mha_fwd(const MhaFwdArgs* args, void* stream);

/* Bytes of workspace mha_fwd needs (0 unless lq is small enough for the split-key kernel). */
size_t mha_fwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dv, int32_t num_splits);

/*
 * Backward pass of tpa_fwd: gradients with respect to the six factor arrays.  Replaces _bwd /
 * _tpa_bwd (tpa/tpa.py:168-214,823-962).  Needs the forward's o and lse.
 */
int tpa_bwd(const TpaBwdArgs* args, void* stream);

/* Bytes of workspace tpa_bwd needs (dense Q, K, V, their gradients and delta, all fp32). */
size_t tpa_bwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv);

/* Backward pass of mha_fwd (tpa/mha.py:40-65). */
int mha_bwd(const MhaBwdArgs* args, void* stream);

/* Bytes of workspace mha_bwd needs (delta; plus fp32 copies of q, k, v when dtype is not fp32). */
size_t mha_bwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t dtype);

#ifdef __cplusplus
}
#endif
#endif /* TPA_ABI_H_ */
