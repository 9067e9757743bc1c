/*
 * pith_hip.h — flat C ABI of libpith_hip.so: MI355X (gfx950) kernels for PithTrain's
 * context-parallel ring-attention hot path.
 *
 * Conventions (all entry points):
 *   - return 0 (PITH_OK) on success, a negative PITH_ERR_* code otherwise; the text of the
 *     last error of the calling thread is available from pith_last_error();
 *   - every pointer is a borrowed DEVICE pointer; the library allocates and frees nothing and
 *     keeps no state between calls; calls only enqueue work on `stream` (a hipStream_t passed
 *     as void*, NULL = the default stream) and never synchronise the device;
 *   - activations are bf16 in BSHD order, x[b, s, h, d] at  b*batch_stride + (s*H + h)*D + d
 *     (strides in ELEMENTS; the row stride H*D and head stride D are implied, which is what
 *     the reference asserts with .is_contiguous(); the separate batch stride lets a caller
 *     pass a slice along S without copying);
 *   - LSE and delta are fp32 in BHS order, lse[b, h, s] at  b*bs + h*hs + s  with both
 *     strides given so that a row sub-range of a [B,H,S] tensor can be addressed in place;
 *   - LSE is base-2 (log2 of the softmax denominator in the scaled-score domain) unless a
 *     `base` field says otherwise.
 *
 * Reference interface replaced (paths relative to the PithTrain tree):
 *   pithtrain/operators/mla/triton.py:552-603        _mla_fwd / _mla_bwd_preprocess / _mla_bwd_dk_dv / _mla_bwd_dq
 *   pithtrain/operators/ring_attention/standard.py:91-93,134-153   flash-attn _flash_attn_forward / _flash_attn_backward call sites
 *   pithtrain/operators/ring_attention/mla.py:27-40  _online_softmax_combine_log2
 *   pithtrain/operators/ring_attention/standard.py:53-66  _online_softmax_combine
 *   pithtrain/models/qwen3_30b_a3b.py:417-421        q_norm / k_norm + apply_rotary_pos_emb (the step before the path)
 *   pithtrain/models/deepseek_v2_lite.py:446-454     rotary embedding + q/k assembly of the MLA layer (the same step there)
 */
#ifndef PITH_HIP_H
#define PITH_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* pith_stream_t; /* hipStream_t */

enum {
  PITH_OK = 0,
  PITH_ERR_NULL_POINTER = -1, /* a required pointer argument is NULL */
  PITH_ERR_BAD_SHAPE = -2,    /* a size is <= 0, or sizes are inconsistent with each other */
  PITH_ERR_BAD_DTYPE = -3,    /* a dtype / base enum is out of range */
  PITH_ERR_UNSUPPORTED = -4,  /* valid request this build has no kernel for (head dims, causal with Sq != Skv) */
  PITH_ERR_MISALIGNED = -5,   /* a pointer or stride breaks the 16-byte vector-access requirement */
  PITH_ERR_LAUNCH = -6        /* the HIP runtime refused the launch */
};

enum { PITH_BF16 = 0, PITH_F32 = 1 };
enum { PITH_BASE_2 = 0, PITH_BASE_E = 1 };

/* Library version: major*10000 + minor*100 + patch. */
int pith_version(void);
/* Text of the last error raised on the calling thread ("" if none). Never NULL. */
const char* pith_last_error(void);
/* Symbolic name of an error code ("PITH_OK", "PITH_ERR_BAD_SHAPE", ...). Never NULL. */
const char* pith_error_name(int code);

/* What the library sees of a device (index as in hipSetDevice): filled from the HIP runtime. The
 * kernels are built for gfx950 only; `supported` is 1 when arch_name starts with "gfx950". */
typedef struct {
  char arch_name[64];
  int32_t compute_units;
  int32_t lds_bytes_per_workgroup;
  int32_t clock_khz;
  int32_t supported;
  int64_t hbm_bytes;
} pith_device_info_t;

int pith_device_info(int device, pith_device_info_t* info);

/* ------------------------------------------------------------------------------------------
 * Online-softmax combine of two partial attention results.
 * Replaces _online_softmax_combine_log2 (ring_attention/mla.py:27-40, base 2) and
 * _online_softmax_combine (ring_attention/standard.py:53-66, base e):
 *     M = max(l1,l2); w1 = beta^(l1-M); w2 = beta^(l2-M)
 *     out = (w1*out1 + w2*out2)/(w1+w2);  lse = M + log_beta(w1+w2)
 * out1/out2 may each be bf16 or fp32 (the running accumulator of the ring is fp32, a chunk
 * result is bf16); `out` is fp32 (what the reference's type promotion yields) or bf16 (used
 * for the last ring step, fusing the reference's final .to(q.dtype), mla.py:78).
 * `out` may alias out1 or out2 when the dtypes match; lse_out may alias lse1 or lse2.
 * D must be a multiple of 8; base pointers and batch strides must keep 16-byte alignment. */
typedef struct {
  const void* out1;
  const float* lse1;
  const void* out2;
  const float* lse2;
  void* out;
  float* lse_out;
  int32_t dtype1, dtype2, dtype_out; /* PITH_BF16 | PITH_F32 */
  int32_t base;                      /* PITH_BASE_2 | PITH_BASE_E */
  int64_t B, S, H, D;
  int64_t out1_bs, out2_bs, out_bs;  /* batch strides of the three O tensors, elements */
  int64_t lse1_bs, lse1_hs;          /* batch / head strides of lse1 */
  int64_t lse2_bs, lse2_hs;
  int64_t lse_out_bs, lse_out_hs;
} pith_combine_args;

int pith_combine(const pith_combine_args* args, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * One chunk attention forward: O = softmax(scale * Q K^T [+ causal mask]) V and the base-2 LSE.
 * Replaces _mla_fwd (mla/triton.py:552-563; kernels :32-93 causal, :274-323 non-causal) and the
 * _flash_attn_forward call at ring_attention/standard.py:91-93 (whose LSE is natural-log:
 * LSE_e = LSE_2 * ln 2).
 * q [B,Sq,Hq,Dqk], k [B,Skv,Hkv,Dqk], v [B,Skv,Hkv,Dv], o [B,Sq,Hq,Dv] bf16; lse [B,Hq,Sq] fp32.
 * Query head h reads kv head h / (Hq/Hkv). causal != 0 masks key j > query i and needs
 * Sq == Skv. Supported (Dqk, Dv): (64,64), (128,128), (192,128). Sq and Skv are arbitrary.
 *
 * Keys in two parts (k_pe != NULL; MLA, Dqk = 192, Dv = 128 only): the layer's key is
 * [k_nope (128 features, per head) | k_pe (64 rotary features, ONE vector per position shared by
 * all heads)], pithtrain/models/deepseek_v2_lite.py:448-454, where the reference materialises it
 * with k_pe broadcast to every head. Here k is then k_nope [B,Skv,Hkv,128] and k_pe [B,Skv,64]
 * (batch stride k_pe_bs, row stride k_pe_rs, elements: it may be a column slice of a wider
 * tensor) is read beside it; results equal those of the assembled key.
 *
 * Merging with a running result (prev_o != NULL): one ring step in one launch. The chunk's
 * attention result is combined with the running result of the same query rows the way
 * _online_softmax_combine_log2(prev_o, lse, o_chunk, lse_chunk) combines them
 * (ring_attention/mla.py:27-40, called per step at mla.py:64-70 / standard.py:95-101): `lse` holds
 * the running base-2 LSE on entry and the merged LSE on return; prev_o [B,Sq,Hq,Dv] is bf16 or
 * fp32 (prev_o_dtype; the reference's running output is fp32 by promotion, mla.py:38); the merged
 * output is written as bf16 to `o` (may be NULL then) and / or as fp32 to acc_o (may be NULL;
 * at least one of the two), and either may be the same memory as prev_o when the dtypes agree.
 * When both are given, o_rows / acc_o_rows ([begin, end) query rows of this call, multiples of 32
 * or Sq; {0, 0} = all rows) restrict which rows each of them receives: a ring step whose first
 * rows see their last merge (bf16 result) while the others go on (fp32 running value) then writes
 * every row once.
 * Saves the chunk result's round trip through memory and the combine launch. Available for head
 * dims (128,128) and (192,128) without a causal mask (in a ring the causal step is the first one
 * and has nothing to merge with); otherwise PITH_ERR_UNSUPPORTED (run pith_attn_fwd, then
 * pith_combine). */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  int64_t B, Sq, Skv, Hq, Hkv, Dqk, Dv;
  int64_t q_bs, k_bs, v_bs, o_bs; /* batch strides, elements */
  int64_t lse_bs, lse_hs;
  float scale;
  int32_t causal;
  const void* k_pe;          /* NULL: k holds all Dqk features */
  int64_t k_pe_bs, k_pe_rs;  /* batch / row strides of k_pe, elements */
  const void* prev_o;        /* NULL: plain forward (o and lse are only written) */
  int64_t prev_o_bs;         /* batch stride of prev_o, elements */
  float* acc_o;              /* merging only: fp32 copy of the merged output, or NULL */
  int64_t acc_o_bs;
  int32_t prev_o_dtype;      /* PITH_BF16 | PITH_F32 */
  int32_t reserved0;         /* keep 0 */
  int64_t o_rows[2];         /* merging: rows that receive o ({0,0} = all) */
  int64_t acc_o_rows[2];     /* merging: rows that receive acc_o ({0,0} = all) */
} pith_attn_fwd_args;

int pith_attn_fwd(const pith_attn_fwd_args* args, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * delta[b,h,s] = sum_d fp32(o[b,s,h,d]) * fp32(dout[b,s,h,d]).
 * Replaces _mla_bwd_preprocess (mla/triton.py:566-574; kernel :101-122). */
typedef struct {
  const void* o;
  const void* dout;
  float* delta;
  int64_t B, S, H, D;
  int64_t o_bs, dout_bs;
  int64_t delta_bs, delta_hs;
} pith_attn_delta_args;

int pith_attn_bwd_delta(const pith_attn_delta_args* args, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * One chunk attention backward against an EXTERNAL (ring-combined) base-2 LSE and delta:
 *     P = exp2(scale*log2(e)*S - lse);  dV = P^T dO;  dP = dO V^T;
 *     dS = P o (dP - delta) * scale;    dK = dS^T Q;  dQ = dS K
 * Replaces _mla_bwd_dk_dv / _mla_bwd_dq (mla/triton.py:577-603; kernels :130-197, :205-266 and
 * the non-causal twins :331-441) and the _flash_attn_backward call at
 * ring_attention/standard.py:134-153.
 * Shapes as in pith_attn_fwd_args; dout [B,Sq,Hq,Dv] bf16; lse, delta [B,Hq,Sq] fp32.
 * dq [B,Sq,Hq,Dqk], dk [B,Skv,Hkv,Dqk], dv [B,Skv,Hkv,Dv] in dq_dtype / dkv_dtype
 * (PITH_BF16 as the reference stores them, or PITH_F32 for a ring-level accumulator).
 * accumulate_dq != 0 adds to the existing contents of dq instead of overwriting (the ring's
 * `dq += dq_s`, ring_attention/mla.py:116, done in the kernel epilogue); the same for
 * accumulate_dkv. With Hq > Hkv, dk/dv of a kv head sum over its Hq/Hkv query heads.
 * pith_attn_bwd_dkdv ignores dq; pith_attn_bwd_dq ignores dk, dv.
 *
 * Keys in two parts (k_pe != NULL, see pith_attn_fwd_args; needs Hq == Hkv): k and dk are
 * [B,Skv,Hkv,128] (the nope part and its gradient); dk_pe [B,Skv,64] (batch stride dk_pe_bs,
 * contiguous rows, dkv_dtype) receives the gradient of the shared rotary part, i.e. the sum over
 * heads of the last 64 features of the assembled key's gradient, added in head order through the
 * workspace (required then: pith_attn_bwd_dkdv_workspace_bytes).
 *
 * A head range of wider tensors (q_row_heads / kv_row_heads != 0): the call works on Hq (Hkv)
 * CONSECUTIVE heads of tensors whose rows hold q_row_heads (kv_row_heads) heads; q, dout, dq
 * (k, v, dk, dv) point at the first head of the range, row strides are q_row_heads*D
 * (kv_row_heads*D) elements, and lse / delta are addressed through their head stride as always.
 * Results equal the corresponding heads of a call on all heads. This is how a caller bounds the
 * dS hand-over buffer below: one kv head (and its query heads) at a time through one small buffer.
 * Not available together with k_pe.
 *
 * Two ring conveniences that save separate launches (no counterpart in the reference, which runs
 * `torch.zeros_like` per step and adds bf16 partial dQ, standard.py:131-133, mla.py:103,116):
 *   dkv_zero_tail: pith_attn_bwd_dkdv also sets rows [Skv, Skv + dkv_zero_tail) of dk and dv to
 *     zero (not dk_pe; ignored with accumulate_dkv): the rows of a chunk that a zigzag step does not
 *     see owe a zero gradient.
 *   dq_final (pith_attn_bwd_dq, dq_dtype PITH_F32, head dims (128,128) or (192,128)): query rows
 *     [dq_final_rows[0], dq_final_rows[1]) (multiples of 32 or Sq; {0,0} = all) receive their
 *     result - the old contents of dq included when accumulate_dq is set - rounded to bf16 in
 *     dq_final [B,Sq,Hq,Dqk] (laid out like dq) instead of dq: the last ring step that touches a row
 *     range emits the final bf16 gradient, and no cast pass over the fp32 accumulator is needed. */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  const void* dout;
  const float* lse;
  const float* delta;
  void* dq;
  void* dk;
  void* dv;
  int64_t B, Sq, Skv, Hq, Hkv, Dqk, Dv;
  int64_t q_bs, k_bs, v_bs, dout_bs;
  int64_t dq_bs, dk_bs, dv_bs;
  int64_t lse_bs, lse_hs;     /* strides shared by lse and delta */
  float scale;
  int32_t causal;
  int32_t dq_dtype, dkv_dtype;
  int32_t accumulate_dq, accumulate_dkv;
  void* workspace;         /* optional device scratch for pith_attn_bwd_dkdv, 16-byte aligned; may be NULL */
  int64_t workspace_bytes; /* its size */
  const void* k_pe;          /* NULL: k holds all Dqk features */
  int64_t k_pe_bs, k_pe_rs;  /* batch / row strides of k_pe, elements */
  void* dk_pe;               /* pith_attn_bwd_dkdv with k_pe: gradient of k_pe */
  int64_t dk_pe_bs;
  void* ds;                  /* optional dS hand-over buffer (see below), 256-byte aligned; may be NULL */
  int64_t ds_bytes;          /* its size */
  int64_t q_row_heads;       /* heads per row of q, dout, dq (0 = Hq) */
  int64_t kv_row_heads;      /* heads per row of k, v, dk, dv (0 = Hkv) */
  int64_t dkv_zero_tail;     /* rows behind the Skv rows of dk, dv to clear (0 = none) */
  void* dq_final;            /* bf16 destination of finished dQ rows, or NULL */
  int64_t dq_final_bs;       /* its batch stride, elements */
  int64_t dq_final_rows[2];  /* query rows that go to dq_final ({0,0} = all) */
} pith_attn_bwd_args;

int pith_attn_bwd_dkdv(const pith_attn_bwd_args* args, pith_stream_t stream);
int pith_attn_bwd_dq(const pith_attn_bwd_args* args, pith_stream_t stream);

/* Scratch size with which pith_attn_bwd_dkdv runs fastest for these shapes (0 = none needed).
 * With grouped-query attention and few key rows the kernel spreads the query heads of a group
 * over several workgroups, which leave fp32 partial dK/dV in the workspace; a second kernel adds
 * them in a fixed order (results do not depend on scheduling). Without a workspace, or with a
 * smaller one, the call still succeeds and one workgroup walks all heads of a group. The
 * workspace is only used during the call's kernels; nothing is kept in it between calls. */
int64_t pith_attn_bwd_dkdv_workspace_bytes(const pith_attn_bwd_args* args);

/* dS hand-over between the two backward calls of one chunk (no counterpart in the reference, whose
 * two kernels each recompute S and dP, mla/triton.py:130-266). When `ds` is set,
 * pith_attn_bwd_dkdv also stores every dS tile it forms (bf16, in a layout private to the library)
 * and a pith_attn_bwd_dq call with the SAME shapes, strides, causal flag and `ds`, enqueued after
 * it on the same stream, computes dQ = scale * dS K from those tiles without recomputing the
 * scores: the backward then executes 5 matrix products instead of 7, at the price of
 * Sq*Skv*Hq*B*2 bytes written and read once (a causal call keeps only the tiles at or below the
 * diagonal: about half). Results agree with the recomputing dQ kernel up to
 * fp32 summation order (the dS values are the same bf16 numbers). The buffer holds nothing of
 * value after the dQ call. Returns the bytes needed, or 0 when the shape has no hand-over path
 * (head dims other than (128,128)); with ds == NULL or a buffer that is too small both calls
 * behave as before. */
int64_t pith_attn_bwd_ds_bytes(const pith_attn_bwd_args* args);

/* pith_attn_bwd_dkdv for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the
 * reference. Same arguments and results, bit for bit, as pith_attn_bwd_dkdv called with a
 * workspace of pith_attn_bwd_dkdv_workspace_bytes() bytes, but `workspace` / `workspace_bytes`
 * are ignored: the head-split partial sums go to a scratch array that is part of the library's
 * code object (PITH_DKDV_STATIC_SCRATCH_BYTES of device memory on every GPU the library runs on,
 * held until the process ends). The call allocates and frees nothing. A shape whose partial sums
 * need more than the scratch holds is rejected with PITH_ERR_UNSUPPORTED. The first call on a
 * device looks up the array's device address (make it outside a graph capture). All calls on
 * one GPU share that GPU's array: calls that may overlap in time (different streams, different
 * threads) race and must be ordered by the caller. */
#define PITH_DKDV_STATIC_SCRATCH_BYTES (64ll << 20)
int pith_attn_bwd_dkdv_static(const pith_attn_bwd_args* args, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * dst[i] = bf16(src[i]) with round-to-nearest-even, i < n. Replaces the reference's
 * `.to(q.dtype)` on an fp32 accumulator (ring_attention/mla.py:78, standard.py:104) when the
 * last combine did not already emit bf16. n must be a multiple of 8. */
int pith_cast_f32_bf16(const float* src, void* dst, int64_t n, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Attention prologue of the GQA layer: per-head RMSNorm followed by the rotary embedding,
 *     y   = x * rsqrt(mean_d(x^2) + eps) * weight          (each [b, s, h] row of D elements)
 *     out = y * cos + rotate_half(y) * sin,  rotate_half(y) = cat(-y[D/2:], y[:D/2])
 * Replaces q_norm / k_norm (torch.nn.RMSNorm over the head dim) and apply_rotary_pos_emb at
 * pithtrain/models/qwen3_30b_a3b.py:417-421 (definitions :100-136, :381-382); called once for q
 * and once for k. weight == NULL skips the normalisation (apply_rotary_pos_emb alone).
 * x, out, dout [B,S,H,D] bf16; cos, sin [B,S,D] bf16 with batch stride cs_bs (0 = one [S,D]
 * table shared by all batch elements); weight [D] bf16 or fp32. Arithmetic is fp32 with one
 * rounding to bf16 at the end. D must be 8 * a power of two, at most 512; pointers and batch
 * strides must keep 8-byte alignment. `out` may alias x (forward) or dout (backward).
 * Backward: `out` receives dx; with a weight, dweight [D] fp32 is overwritten with the sum over
 * all rows, added in a fixed order through `workspace` (size from
 * pith_norm_rope_bwd_workspace_bytes; required then). The forward ignores dout, dweight and the
 * workspace. */
typedef struct {
  const void* x;
  const void* weight;
  const void* cos;
  const void* sin;
  const void* dout;
  void* out;
  float* dweight;
  void* workspace;
  int64_t workspace_bytes;
  int64_t B, S, H, D;
  int64_t x_bs, out_bs, dout_bs, cs_bs; /* batch strides, elements */
  float eps;
  int32_t weight_dtype; /* PITH_BF16 | PITH_F32 */
} pith_norm_rope_args;

int pith_norm_rope_fwd(const pith_norm_rope_args* args, pith_stream_t stream);
int pith_norm_rope_bwd(const pith_norm_rope_args* args, pith_stream_t stream);
int64_t pith_norm_rope_bwd_workspace_bytes(const pith_norm_rope_args* args);

/* The same for two tensors in ONE launch each way: q and k of a layer, which the reference
 * handles together (pithtrain/models/qwen3_30b_a3b.py:417-421). Results are identical to two
 * single-tensor calls. The two argument structs are independent (own H, weight, workspace, even
 * cos/sin) except that B must agree and either both or neither has a weight. */
int pith_norm_rope_fwd_pair(const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream);
int pith_norm_rope_bwd_pair(const pith_norm_rope_args* a, const pith_norm_rope_args* b, pith_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Attention prologue of the MLA layer: rotary embedding of the rope parts and assembly of the
 * attention operands. Replaces pithtrain/models/deepseek_v2_lite.py:446-454 and the
 * value_states.contiguous() of :462/:467 (apply_rotary_pos_emb :173-187, rotate_half :165-169):
 *     pe'  = de-interleave(pe): pe'[j] = pe[2j], pe'[Dr/2+j] = pe[2j+1]
 *     rot(pe) = pe' * cos[pos] + rotate_half(pe') * sin[pos]
 *     q_out = [q[..., :Dn] | rot(q[..., Dn:])]            [B,S,H,Dn+Dr]
 *     k_out = [kv[..., :Dn] | rot(k_pe) for every head]   [B,S,H,Dn+Dr]
 *     v_out = kv[..., Dn:]                                [B,S,H,Dv]
 * q [B,S,H,Dn+Dr] and kv [B,S,H,Dn+Dv] bf16 are contiguous per batch element (batch strides
 * given); k_pe [B,S,Dr] bf16 has a row stride (it is a column slice of a wider projection);
 * cos, sin [P,Dr] bf16 tables indexed by position_ids [B,S] int64 (batch stride pos_bs; NULL =
 * position s). Positions outside [0,P) are clamped. Outputs are contiguous.
 * Backward: dq_out, dk_out, dv_out are the gradients of the three outputs (contiguous); q_out
 * receives dq [B,S,H,Dn+Dr], k_out receives dkv [B,S,H,Dn+Dv], v_out receives dk_pe [B,S,Dr]
 * (summed over heads in head order); q, kv, k_pe are not read.
 * Dn and Dv must be multiples of 8, Dr of 16; pointers and strides keep 16-byte alignment. */
typedef struct {
  const void* q;
  const void* kv;
  const void* k_pe;
  const void* cos;
  const void* sin;
  const int64_t* position_ids;
  void* q_out;
  void* k_out;
  void* v_out;
  const void* dq_out;
  const void* dk_out;
  const void* dv_out;
  int64_t B, S, H, Dn, Dr, Dv, P;
  int64_t q_bs, kv_bs;        /* batch strides, elements */
  int64_t k_pe_bs, k_pe_rs;   /* batch and row strides of k_pe, elements */
  int64_t pos_bs;             /* batch stride of position_ids (0 = shared) */
} pith_mla_assemble_args;

int pith_mla_assemble_fwd(const pith_mla_assemble_args* args, pith_stream_t stream);
int pith_mla_assemble_bwd(const pith_mla_assemble_args* args, pith_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PITH_HIP_H */
