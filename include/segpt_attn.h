/*
 * segpt_attn.h -- C ABI of libsegpt_attn.so: fused QK-norm causal GQA flash
 * attention (forward + backward) for AMD MI355X (gfx950).
 *
 * The library is the device side of a drop-in for the reference's fused op
 *   sample_efficient_gpt/transformer/ops/triton_flash_attn_qknorm.py:262-343
 *   (TritonFlashAttnQKNormFunc) and of the live module it stands in for
 *   sample_efficient_gpt/transformer/attention.py:43-80 (SelfDotProductAttnQKNorm),
 * plus the caller glue the kernels absorb (GQA expansion attention.py:207-218,
 * value-residual mix :222-228, per-head gate :249-255).
 *
 * Conventions
 *   - plain pointers and sizes only; no torch / HIP types in any signature
 *     (`stream` is a hipStream_t passed as void*; NULL = the null stream);
 *   - the caller owns ALL memory (inputs, outputs, workspace); the library never
 *     allocates, frees or keeps device pointers past a call, and never
 *     synchronises: work is enqueued on `stream` and the call returns;
 *   - return value: 0 ok; < 0 argument / unsupported-shape error detected before
 *     any launch (SEGPT_E_*); > 0 a hipError_t raised by a launch;
 *   - re-entrant: no mutable global state (except segpt_attn_fwd_noalloc, whose calls share one device scratch
 *     array per GPU: see its comment).
 *
 * Mathematics (per batch b, query head h, kv head g = h / (H/Hkv)):
 *   a_i = rsqrt(mean_d q_i^2 + eps)      b_j = rsqrt(mean_d k_j^2 + eps)
 *   s_ij = sm_scale * sum_d (a_i q_id g_q[d]) (b_j k_jd g_k[d]),  j <= i + q_start if causal
 *   v'_j = c1 v_j + c2 v_first_j         (if vr_coef != NULL, (c1,c2) = vr_coef[0..1])
 *   lse_i = log sum_j exp s_ij ;  o_i = sum_j exp(s_ij - lse_i) v'_j
 *   y_i = gate_scale * sigmoid(gate[b,i,h]) * o_i   (if gate.ptr != NULL; else y = o)
 * With g_q = gain (1 element), g_k absent, eps = 1e-6, sm_scale = 1/sqrt(D) this is
 * attention.py:51-80; eps = 1e-8/D, sm_scale = 1/D gives triton_flash_attn_qknorm.py:67-91.
 */
#ifndef SEGPT_ATTN_H
#define SEGPT_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SEGPT_ABI_VERSION 2

/* element type of q/k/v/o/gate and their gradients */
#define SEGPT_DTYPE_BF16 0 /* MFMA path: D in {64, 128}                       */
#define SEGPT_DTYPE_FP32 1 /* fp32 FMA path (1e-5 parity): D in {32, 64, 128} */

/* error codes (negative); segpt_strerror() gives the text */
#define SEGPT_OK 0
#define SEGPT_E_NULL -1        /* a required pointer is NULL                                */
#define SEGPT_E_STRUCT -2      /* struct_bytes does not match this library's layout         */
#define SEGPT_E_DTYPE -3       /* unknown dtype                                             */
#define SEGPT_E_SHAPE -4       /* B,H,Hkv,Sq,Sk <= 0, H % Hkv != 0, or numel of a scale     */
#define SEGPT_E_HEAD_DIM -5    /* D not supported for this dtype                            */
#define SEGPT_E_STRIDE -6      /* a stride is negative / misaligned (rows must be 16 B aligned) */
#define SEGPT_E_WORKSPACE -7   /* workspace NULL or smaller than segpt_attn_workspace_bytes */
#define SEGPT_E_EXTRAS -8      /* v_first without vr_coef or the reverse; missing grad slot */
#define SEGPT_E_QSTART -9      /* q_start < 0                                               */
#define SEGPT_E_ALIGN -10      /* a base pointer is not 16-byte aligned                     */
#define SEGPT_E_ROPE -12       /* rope tables: one NULL, misaligned, or too short for the positions */
#define SEGPT_E_STAGE -11      /* unknown stage passed to segpt_attn_bwd_stage              */
#define SEGPT_E_SCRATCH_LIMIT -13 /* segpt_attn_fwd_noalloc: shape needs more than SEGPT_NOALLOC_SCRATCH_BYTES */

/* size of the library-owned device scratch behind segpt_attn_fwd_noalloc (per GPU, held for the process lifetime) */
#define SEGPT_NOALLOC_SCRATCH_BYTES (16u << 20)

/* segpt_attn_params.flags */
#define SEGPT_FLAG_KV_PREPARED 1 /* kv_workspace already holds what the key/value pre-pass writes for these k, v,
                                    v_first, vr_coef and eps (e.g. segpt_attn_fwd just ran on it): skip the pre-pass */

#define SEGPT_FLAG_RUNNING_MAX 2 /* bf16 forward: always subtract a running row maximum before exp2, also when the
                                    QK-norm bound on the logits (sm_scale*D*max|g_q g_k|) would allow the raw
                                    exponent; same results up to rounding, slower */

#define SEGPT_FLAG_DECODE 4      /* forward only, no backward will follow on this kv_workspace: a bf16 call with at most
                                    32 query rows per kv head (H/Hkv * Sq, the reference's generation step,
                                    attention.py:191-198) may run the split-key decode kernels, which read k / v /
                                    v_first once, normalise and rotate on the fly and use kv_workspace for partial
                                    results instead of normalised keys */

#define SEGPT_FLAG_NO_NORM 8     /* plain attention: both RMS normalisers are exactly 1 (eps is ignored), so
                                    s_ij = sm_scale * (q_i o g_q) . (k_j o g_k); with g_q = 1 and no g_k this is the
                                    reference's non-QK-norm path, TritonFlashAttnFunc (triton_flash_attn.py:208-297)
                                    and the SDPA call attention.py:233-240.  Logits are then unbounded: the bf16
                                    forward always keeps a running row maximum */

/* which scratch buffer segpt_attn_workspace_bytes() sizes */
#define SEGPT_WS_KV 0  /* kv_workspace: bf16 copies of the normalised keys (and mixed values); forward AND backward */
#define SEGPT_WS_BWD 1 /* workspace: per-row statistics, normalised queries, partial sums; backward only            */

/* the two stages segpt_attn_fwd() runs, in this order */
#define SEGPT_FWD_STAGE_PRE 0  /* bf16: key/value pre-pass (skipped with SEGPT_FLAG_KV_PREPARED); fp32: nothing */
#define SEGPT_FWD_STAGE_ATTN 1 /* the attention kernel: writes o and lse                                         */

/* the four stages segpt_attn_bwd() runs, in this order */
#define SEGPT_BWD_STAGE_PRE 0    /* bf16: key/value pre-pass (skipped with SEGPT_FLAG_KV_PREPARED): normalised
                                    Khat (and V' = c1 v + c2 v_first) into kv_workspace;
                                    fp32: delta = rowsum(dY*Y), dgate and the gate-scaled dO            */
#define SEGPT_BWD_STAGE_DQ 1     /* dQ and the per-workgroup partials of the scale gradient; on the bf16
                                    path also delta, dgate and Qhat for stage 2 (a positive gate factor
                                    is folded into the row statistics; a gate scale <= 0 adds a
                                    gate-scaled copy of dO)                                              */
#define SEGPT_BWD_STAGE_DKDV 2   /* dK, dV (, dV_first, partial sums of d vr_coef); bf16: also dg_q, dg_k from
                                    the partials of stage 1                                              */
#define SEGPT_BWD_STAGE_REDUCE 3 /* d vr_coef from the partials (fp32: also dg_q, dg_k); launches nothing on
                                    the bf16 path without a value residual                               */

/* [B, heads, S, D] tensor view; the D axis is contiguous (stride 1). Strides in ELEMENTS.
 * The reference's `(h b) S D` flatten (attention.py:199) is stride_b = S*D, stride_h = B*S*D;
 * a `b S (h D)` projection slice is stride_b = S*W, stride_h = D, stride_s = W. */
typedef struct segpt_tensor4 {
  void* ptr;
  int64_t stride_b, stride_h, stride_s;
} segpt_tensor4;

/* [B, Sq, H] per-head gate logits view (attention.py:251: attn_gate(x) is `b seq h`). */
typedef struct segpt_tensor3 {
  void* ptr;
  int64_t stride_b, stride_s, stride_h;
} segpt_tensor3;

typedef struct segpt_attn_params {
  uint32_t struct_bytes; /* = sizeof(segpt_attn_params) */
  int32_t dtype;         /* SEGPT_DTYPE_* */
  int32_t B, H, Hkv, Sq, Sk, D;
  int32_t causal;  /* 0 / 1 */
  int32_t q_start; /* causal diagonal shift: key j visible to query i iff j <= i + q_start */
  int32_t gq_numel; /* 1 (scalar gain, attention.py:41) or D */
  int32_t gk_numel; /* 0 (no k scale), 1 or D */
  float eps, sm_scale, gate_scale;
  int32_t flags; /* SEGPT_FLAG_* */

  /* forward operands */
  segpt_tensor4 q;       /* [B,H,Sq,D]   in  */
  segpt_tensor4 k;       /* [B,Hkv,Sk,D] in  */
  segpt_tensor4 v;       /* [B,Hkv,Sk,D] in  */
  segpt_tensor4 v_first; /* [B,Hkv,Sk,D] in, optional (ptr NULL = no value residual) */
  segpt_tensor3 gate;    /* [B,Sq,H]     in, optional (ptr NULL = no gate) */
  segpt_tensor4 o;       /* [B,H,Sq,D]   fwd: out (y, gated if gate);  bwd: in (the saved y) */
  float* lse;            /* [B,H,Sq] contiguous fp32, natural log; fwd: out, bwd: in */
  const float* g_q;      /* [gq_numel] fp32 device */
  const float* g_k;      /* [gk_numel] fp32 device or NULL */
  const float* vr_coef;  /* [2] fp32 device (c1, c2) or NULL */

  /* backward operands (ignored by segpt_attn_fwd) */
  segpt_tensor4 d_o;      /* [B,H,Sq,D]   in: dL/dy */
  segpt_tensor4 dq;       /* [B,H,Sq,D]   out */
  segpt_tensor4 dk;       /* [B,Hkv,Sk,D] out */
  segpt_tensor4 dv;       /* [B,Hkv,Sk,D] out */
  segpt_tensor4 dv_first; /* [B,Hkv,Sk,D] out, required iff v_first */
  segpt_tensor3 dgate;    /* [B,Sq,H]     out, required iff gate */
  float* dg_q;            /* [gq_numel] fp32 out */
  float* dg_k;            /* [gk_numel] fp32 out, required iff g_k */
  float* dvr_coef;        /* [2] fp32 out, required iff vr_coef */

  void* workspace; /* backward only: >= segpt_attn_workspace_bytes(p, SEGPT_WS_BWD), 256 B aligned; contents
                      undefined on entry */
  size_t workspace_bytes;
  void* kv_workspace; /* bf16 forward and backward: >= segpt_attn_workspace_bytes(p, SEGPT_WS_KV), 256 B aligned.
                         Written by the key/value pre-pass of either call; a backward that gets the buffer its
                         forward used may set SEGPT_FLAG_KV_PREPARED.  Ignored (may be NULL) for fp32. */
  size_t kv_workspace_bytes;

  /* optional rotary embedding of q and k, fused into the loads (the step before the op in the reference:
   * rope.py:36-56 applied at attention.py:202-204).  Split-half pairs (j, j + D/2); query row i uses table row
   * rope_q_pos0 + i, key row j uses rope_k_pos0 + j.  Both tables or neither.  dq / dk are
   * gradients with respect to the UNROTATED inputs. */
  const float* rope_cos; /* [rope_len, D/2] fp32 device, 16 B aligned, or NULL */
  const float* rope_sin; /* [rope_len, D/2] fp32 device, 16 B aligned, or NULL */
  int32_t rope_len;
  int32_t rope_q_pos0; /* the reference passes q_start here (attention.py:191-195) */
  int32_t rope_k_pos0;
  int32_t reserved0;
} segpt_attn_params;

/* ABI revision of the loaded library (compare with SEGPT_ABI_VERSION). No reference counterpart. */
int segpt_abi_version(void);

/* Static text for a return code of this library (negative) or "hip error" class (positive).
 * Replaces the Python AssertionErrors of triton_flash_attn_qknorm.py:273-276. */
const char* segpt_strerror(int code);

/* Bytes of device scratch of kind `which` (SEGPT_WS_*) these params need (0 is possible). Validates
 * nothing but sizes; returns 0 for invalid params (the launch call will report the error).
 * SEGPT_WS_KV follows p->flags: a decode-shaped forward with SEGPT_FLAG_DECODE needs only the split-key partial
 * results (a small fraction of the cache), every other call the normalised keys (and mixed values).
 * Replaces the in-op allocations of triton_flash_attn_qknorm.py:286-287 / :320-323: the caller
 * allocates. */
size_t segpt_attn_workspace_bytes(const segpt_attn_params* p, int which);

/* Forward: writes o (y) and lse (bf16: and kv_workspace).  Replaces the launch
 * `flashatt_qknorm_kernel_fwd[grid](...)`, triton_flash_attn_qknorm.py:290-302 (kernel :22-115),
 * and in the live path the normalise + SDPA sequence attention.py:52-80. */
int segpt_attn_fwd(const segpt_attn_params* p, void* stream);

/* Backward: reads q,k,v,(v_first,gate),o,lse,d_o; writes dq,dk,dv,(dv_first,dgate),dg_q,(dg_k,dvr_coef).
 * Deterministic (no floating-point atomics).  Replaces the launch
 * `flashatt_qknorm_kernel_bwd[grid](...)`, triton_flash_attn_qknorm.py:326-342 (kernel :125-255). */
int segpt_attn_bwd(const segpt_attn_params* p, void* stream);

/* One launch of the backward, for profilers and benchmarks that time the kernels separately:
 * segpt_attn_bwd(p, s) is exactly stages 0, 1, 2, 3 in this order on one stream with the same params
 * and workspace.  Each stage needs the earlier ones to have run on the same workspace.  No counterpart in the
 * reference (its backward is the single kernel triton_flash_attn_qknorm.py:125-255). */
int segpt_attn_bwd_stage(const segpt_attn_params* p, int stage, void* stream);

/* The same for the forward: segpt_attn_fwd(p, s) is stages SEGPT_FWD_STAGE_PRE, SEGPT_FWD_STAGE_ATTN in this
 * order.  No counterpart in the reference (its forward is the single kernel triton_flash_attn_qknorm.py:22-115). */
int segpt_attn_fwd_stage(const segpt_attn_params* p, int stage, void* stream);

/* segpt_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same operands and results as
 * segpt_attn_fwd, except that p->kv_workspace / kv_workspace_bytes are ignored: the key/value scratch (normalised
 * keys and mixed values, or the split-key partial results of a SEGPT_FLAG_DECODE call) is a fixed
 * SEGPT_NOALLOC_SCRATCH_BYTES array inside the library's device image.  The call allocates and frees nothing;
 * a shape whose segpt_attn_workspace_bytes(p, SEGPT_WS_KV) exceeds the array returns SEGPT_E_SCRATCH_LIMIT
 * before any launch.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race, and no later call may rely on its contents (SEGPT_FLAG_KV_PREPARED is ignored here, and
 * a backward must run its own key/value pre-pass on a caller-owned kv_workspace).
 * The array that is used is the CURRENT device's (hipGetDevice), so `stream` must be a stream of the current device
 * (another device's stream returns hipErrorInvalidDevice).  The first call on each device looks the array's address
 * up (hipGetSymbolAddress) and keeps it: make that first call outside stream capture; later calls are plain kernel
 * launches and may be captured into a HIP graph and replayed.  The array is part of the library's device image and
 * occupies its SEGPT_NOALLOC_SCRATCH_BYTES on every GPU the library is loaded on, used or not. */
int segpt_attn_fwd_noalloc(const segpt_attn_params* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SEGPT_ATTN_H */
