// C ABI of libsegpt_attn.so: argument validation, workspace carve-up and dispatch.
// No device memory is allocated or freed here; nothing synchronises.
#include <mutex>

#include "common.hpp"

// Scratch of segpt_attn_fwd_noalloc(): lives in the library's device image, one copy per GPU the library runs on,
// held until the process ends.  In host code this name is only a handle for hipGetSymbolAddress(); kernels and
// copies get the per-device address looked up below.
static __device__ __align__(256) unsigned char scratch[SEGPT_NOALLOC_SCRATCH_BYTES];

namespace segpt {

int f32_rows_per_block();
int bf16_dq_grid(const segpt_attn_params& p);
int bf16_dkdv_grid(const segpt_attn_params& p);

int dq_blocks(const segpt_attn_params& p) {
  if (p.dtype != SEGPT_DTYPE_FP32) return bf16_dq_grid(p);
  const int rows = f32_rows_per_block();
  return ((p.Sq + rows - 1) / rows) * p.H * p.B;
}
int dkdv_blocks(const segpt_attn_params& p) {
  if (p.dtype != SEGPT_DTYPE_FP32) return bf16_dkdv_grid(p);
  const int rows = f32_rows_per_block();
  return ((p.Sk + rows - 1) / rows) * p.Hkv * p.B;
}

namespace {

size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }
size_t elem_bytes(const segpt_attn_params& p) { return p.dtype == SEGPT_DTYPE_FP32 ? 4 : 2; }

struct WsLayout {
  size_t delta, nlse2, do_eff, qhat, dg_part, dcoef_part, total;
};
struct KvLayout {
  size_t khat, vmix, total;
};

// A forward-only bf16 call with at most 32 query rows per kv head takes the split-key decode kernels when the
// caller allows it with SEGPT_FLAG_DECODE; the kv workspace then holds partial results, not keys.
bool decode_shape(const segpt_attn_params& p) {
  return (p.flags & SEGPT_FLAG_DECODE) && p.dtype == SEGPT_DTYPE_BF16 && p.Hkv > 0 && (int64_t)(p.H / p.Hkv) * p.Sq <= 32;
}

// bf16 only: normalised keys and (with a value residual) mixed values, contiguous [B,Hkv,Sk,D]; for a decode-shaped
// call the per-split partial results instead (a small fraction of the cache)
KvLayout kv_layout(const segpt_attn_params& p) {
  KvLayout w{0, 0, 0};
  if (p.dtype != SEGPT_DTYPE_BF16) return w;
  if (decode_shape(p)) {
    int kend, splits, chunk;
    w.total = align_up(decode_plan(p, &kend, &splits, &chunk));
    return w;
  }
  const size_t kvrows = (size_t)p.B * p.Hkv * p.Sk;
  size_t off = align_up(kvrows * p.D * 2);
  w.vmix = off;
  if (p.v_first.ptr) off += align_up(kvrows * p.D * 2);
  w.total = off;
  return w;
}

// The backward keeps a gate-scaled copy of dO on the fp32 path and, on the bf16 path, only for a gate scale that is
// not positive: a positive gate factor travels to the dK/dV kernel inside the two row statistics instead.
bool gated_do_copy(const segpt_attn_params& p) {
  return p.gate.ptr && (p.dtype == SEGPT_DTYPE_FP32 || !(p.gate_scale > 0.f));
}

WsLayout bwd_layout(const segpt_attn_params& p) {
  WsLayout w;
  size_t off = 0;
  const size_t rows = (size_t)p.B * p.H * p.Sq;
  w.delta = off;
  off += align_up(rows * sizeof(float));
  w.nlse2 = off;
  if (p.dtype == SEGPT_DTYPE_BF16) off += align_up(rows * sizeof(float));
  w.do_eff = off;
  if (gated_do_copy(p)) off += align_up(rows * p.D * elem_bytes(p));
  w.qhat = off;
  if (p.dtype == SEGPT_DTYPE_BF16) off += align_up(rows * p.D * 2);
  w.dg_part = off;
  off += align_up((size_t)dq_blocks(p) * p.D * sizeof(float));
  w.dcoef_part = off;
  off += align_up((size_t)dkdv_blocks(p) * 2 * sizeof(float));
  w.total = off;
  return w;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

int check_t4(const segpt_tensor4& t, const segpt_attn_params& p) {
  if (!t.ptr) return SEGPT_E_NULL;
  if (!aligned16(t.ptr)) return SEGPT_E_ALIGN;
  const int64_t per16 = 16 / (int64_t)elem_bytes(p);
  if (t.stride_b < 0 || t.stride_h < 0 || t.stride_s < p.D) return SEGPT_E_STRIDE;
  if (t.stride_b % per16 || t.stride_h % per16 || t.stride_s % per16) return SEGPT_E_STRIDE;
  // the bf16 kernels address the rows of a tile (up to 256 of them) by 32-bit byte offsets from the tile's first row
  if (p.dtype == SEGPT_DTYPE_BF16 && t.stride_s > (int64_t)(UINT32_MAX / (256 * 2))) return SEGPT_E_STRIDE;
  return SEGPT_OK;
}

// An OUTPUT view must not alias itself: with the extents (B, heads, rows) sorted by stride, every stride has to
// step over the whole extent below it (a zero or too-small stride would make workgroups race on the same rows and
// the call would still report success).  Extents of 1 are free.
int check_t4_out(const segpt_tensor4& t, const segpt_attn_params& p, int heads, int rows) {
  const int rc = check_t4(t, p);
  if (rc) return rc;
  int64_t st[3] = {t.stride_b, t.stride_h, t.stride_s};
  int64_t ex[3] = {p.B, heads, rows};
  for (int i = 0; i < 3; ++i)
    for (int j = i + 1; j < 3; ++j)
      if (st[j] < st[i]) { const int64_t a = st[i], b = ex[i]; st[i] = st[j]; ex[i] = ex[j]; st[j] = a; ex[j] = b; }
  int64_t span = p.D;  // elements covered by everything below the current dimension
  for (int i = 0; i < 3; ++i) {
    if (ex[i] <= 1) continue;
    if (st[i] < span) return SEGPT_E_STRIDE;
    span = st[i] * ex[i];
  }
  return SEGPT_OK;
}

int check_common(const segpt_attn_params* p) {
  if (!p) return SEGPT_E_NULL;
  if (p->struct_bytes != sizeof(segpt_attn_params)) return SEGPT_E_STRUCT;
  if (p->dtype != SEGPT_DTYPE_BF16 && p->dtype != SEGPT_DTYPE_FP32) return SEGPT_E_DTYPE;
  if (p->B <= 0 || p->H <= 0 || p->Hkv <= 0 || p->Sq <= 0 || p->Sk <= 0) return SEGPT_E_SHAPE;
  if (p->H % p->Hkv != 0) return SEGPT_E_SHAPE;
  if (p->B > 65535 || p->H > 65535) return SEGPT_E_SHAPE;
  if (p->dtype == SEGPT_DTYPE_BF16) {
    if (p->D != 64 && p->D != 128) return SEGPT_E_HEAD_DIM;
  } else {
    if (p->D != 32 && p->D != 64 && p->D != 128) return SEGPT_E_HEAD_DIM;
  }
  if (p->gq_numel != 1 && p->gq_numel != p->D) return SEGPT_E_SHAPE;
  if (p->gk_numel != 0 && p->gk_numel != 1 && p->gk_numel != p->D) return SEGPT_E_SHAPE;
  if (p->q_start < 0) return SEGPT_E_QSTART;
  if (!p->g_q || !p->lse) return SEGPT_E_NULL;
  if ((p->gk_numel != 0) != (p->g_k != nullptr)) return SEGPT_E_SHAPE;
  if ((p->v_first.ptr != nullptr) != (p->vr_coef != nullptr)) return SEGPT_E_EXTRAS;
  int rc;
  if ((rc = check_t4(p->q, *p))) return rc;
  if ((rc = check_t4(p->k, *p))) return rc;
  if ((rc = check_t4(p->v, *p))) return rc;
  if (p->v_first.ptr && (rc = check_t4(p->v_first, *p))) return rc;
  if (p->gate.ptr && (p->gate.stride_b < 0 || p->gate.stride_s < 0 || p->gate.stride_h < 0)) return SEGPT_E_STRIDE;
  if (p->rope_cos || p->rope_sin) {
    if (!p->rope_cos || !p->rope_sin) return SEGPT_E_ROPE;
    if (!aligned16(p->rope_cos) || !aligned16(p->rope_sin)) return SEGPT_E_ROPE;
    if (p->rope_q_pos0 < 0 || p->rope_k_pos0 < 0) return SEGPT_E_ROPE;
    if ((int64_t)p->rope_q_pos0 + p->Sq > p->rope_len || (int64_t)p->rope_k_pos0 + p->Sk > p->rope_len) return SEGPT_E_ROPE;
  }
  if (p->dtype == SEGPT_DTYPE_BF16) {
    if (!p->kv_workspace || p->kv_workspace_bytes < kv_layout(*p).total) return SEGPT_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(p->kv_workspace) & 255u) return SEGPT_E_ALIGN;
  }
  return SEGPT_OK;
}

// fills the kernel arguments that both directions share
void bind_kv(KArgs& a) {
  const segpt_attn_params& p = a.p;
  if (p.dtype != SEGPT_DTYPE_BF16) return;
  const KvLayout kv = kv_layout(p);
  char* ws = reinterpret_cast<char*>(p.kv_workspace);
  a.khat = reinterpret_cast<uint16_t*>(ws + kv.khat);
  a.vmix = p.v_first.ptr ? reinterpret_cast<uint16_t*>(ws + kv.vmix) : nullptr;
}

int check_bwd(const segpt_attn_params* p) {
  int rc;
  if ((rc = check_t4(p->o, *p))) return rc;  // the saved output: an input here
  if ((rc = check_t4(p->d_o, *p))) return rc;
  if ((rc = check_t4_out(p->dq, *p, p->H, p->Sq))) return rc;
  if ((rc = check_t4_out(p->dk, *p, p->Hkv, p->Sk))) return rc;
  if ((rc = check_t4_out(p->dv, *p, p->Hkv, p->Sk))) return rc;
  if (!p->dg_q) return SEGPT_E_NULL;
  if (p->g_k && !p->dg_k) return SEGPT_E_EXTRAS;
  if (p->v_first.ptr) {
    if (!p->dv_first.ptr || !p->dvr_coef) return SEGPT_E_EXTRAS;
    if ((rc = check_t4_out(p->dv_first, *p, p->Hkv, p->Sk))) return rc;
  }
  if (p->gate.ptr) {
    if (!p->dgate.ptr) return SEGPT_E_EXTRAS;
    if (p->dgate.stride_b < 0 || p->dgate.stride_s < 0 || p->dgate.stride_h < 0) return SEGPT_E_STRIDE;
  }
  const WsLayout w = bwd_layout(*p);
  if (!p->workspace || p->workspace_bytes < w.total) return SEGPT_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(p->workspace) & 255u) return SEGPT_E_ALIGN;
  return SEGPT_OK;
}

}  // namespace
}  // namespace segpt

using namespace segpt;

extern "C" {

int segpt_abi_version(void) { return SEGPT_ABI_VERSION; }

const char* segpt_strerror(int code) {
  switch (code) {
    case SEGPT_OK: return "ok";
    case SEGPT_E_NULL: return "a required pointer is NULL";
    case SEGPT_E_STRUCT: return "segpt_attn_params.struct_bytes does not match this library (ABI mismatch)";
    case SEGPT_E_DTYPE: return "unknown dtype (expected SEGPT_DTYPE_BF16 or SEGPT_DTYPE_FP32)";
    case SEGPT_E_SHAPE: return "bad shape: sizes must be positive, H divisible by Hkv, scale vectors of 1 or D elements";
    case SEGPT_E_HEAD_DIM: return "unsupported head_dim: bf16 needs D in {64,128}, fp32 D in {32,64,128}";
    case SEGPT_E_STRIDE: return "bad stride: strides must be non-negative multiples of 16 bytes, rows must not overlap, and a bf16 row stride must stay below 2^23 elements";
    case SEGPT_E_WORKSPACE: return "workspace or kv_workspace missing or smaller than segpt_attn_workspace_bytes()";
    case SEGPT_E_EXTRAS: return "inconsistent optional operands (v_first/vr_coef/gate and their gradient slots)";
    case SEGPT_E_QSTART: return "q_start must be >= 0";
    case SEGPT_E_ALIGN: return "a base pointer is not 16-byte aligned (workspace: 256-byte)";
    case SEGPT_E_ROPE: return "rope tables: both or neither, 16-byte aligned, rope_len >= position + rows";
    case SEGPT_E_STAGE: return "unknown stage (expected SEGPT_FWD_STAGE_* / SEGPT_BWD_STAGE_*)";
    case SEGPT_E_SCRATCH_LIMIT: return "segpt_attn_fwd_noalloc: the key/value scratch this shape needs exceeds SEGPT_NOALLOC_SCRATCH_BYTES";
    default: return code > 0 ? "HIP runtime error raised by a kernel launch" : "unknown segpt error code";
  }
}

size_t segpt_attn_workspace_bytes(const segpt_attn_params* p, int which) {
  if (!p || p->struct_bytes != sizeof(segpt_attn_params)) return 0;
  if (p->B <= 0 || p->H <= 0 || p->Hkv <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->D <= 0) return 0;
  if (p->dtype == SEGPT_DTYPE_BF16 && p->D != 64 && p->D != 128) return 0;
  if (which == SEGPT_WS_KV) return kv_layout(*p).total;
  if (which == SEGPT_WS_BWD) return bwd_layout(*p).total;
  return 0;
}

static bool use_decode(const segpt_attn_params* p) { return decode_shape(*p); }  // check_common sized the workspace for it

static int fwd_stage_impl(const segpt_attn_params* p, int stage_lo, int stage_hi, void* stream) {
  int rc = check_common(p);
  if (rc) return rc;
  if ((rc = check_t4_out(p->o, *p, p->H, p->Sq))) return rc;
  KArgs a{};
  a.p = *p;
  bind_kv(a);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool f32 = p->dtype == SEGPT_DTYPE_FP32;
  const bool decode = use_decode(p);
  for (int stage = stage_lo; stage <= stage_hi; ++stage) {
    switch (stage) {
      case SEGPT_FWD_STAGE_PRE: rc = (f32 || decode || (p->flags & SEGPT_FLAG_KV_PREPARED)) ? 0 : launch_kv_prep(a, st); break;
      case SEGPT_FWD_STAGE_ATTN: rc = f32 ? launch_fwd_f32(a, st) : (decode ? launch_fwd_decode_bf16(a, st) : launch_fwd_bf16(a, st)); break;
      default: return SEGPT_E_STAGE;
    }
    if (rc) return rc;
  }
  return SEGPT_OK;
}

int segpt_attn_fwd(const segpt_attn_params* p, void* stream) {
  return fwd_stage_impl(p, SEGPT_FWD_STAGE_PRE, SEGPT_FWD_STAGE_ATTN, stream);
}

// Device address of `scratch` on the CURRENT device, looked up once per device (first call there).  Kernels are
// launched on `stream`, so the stream has to belong to the current device: a stream of another GPU would run them
// against this GPU's copy of the array, and is refused.
static int noalloc_scratch_ptr(void** out, hipStream_t stream) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
  if (stream) {  // the null stream is the current device's by definition
    hipDevice_t sdev = -1;
    if (hipStreamGetDevice(stream, &sdev) == hipSuccess && (int)sdev != dev) return (int)hipErrorInvalidDevice;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    ptrs[dev] = ptr;
  }
  *out = ptrs[dev];
  return 0;
}

int segpt_attn_fwd_noalloc(const segpt_attn_params* p, void* stream) {
  if (!p) return SEGPT_E_NULL;
  if (p->struct_bytes != sizeof(segpt_attn_params)) return SEGPT_E_STRUCT;
  segpt_attn_params q = *p;
  q.kv_workspace = nullptr;
  q.kv_workspace_bytes = 0;
  q.flags &= ~SEGPT_FLAG_KV_PREPARED;  // the scratch is shared by every call on this GPU: never assume its contents
  if (q.dtype == SEGPT_DTYPE_BF16) {
    if (segpt_attn_workspace_bytes(&q, SEGPT_WS_KV) > (size_t)SEGPT_NOALLOC_SCRATCH_BYTES) return SEGPT_E_SCRATCH_LIMIT;
    // argument errors first (they need no device): validate against a stand-in address, then look the real one up
    q.kv_workspace = reinterpret_cast<void*>(uintptr_t{256});
    q.kv_workspace_bytes = SEGPT_NOALLOC_SCRATCH_BYTES;
    int rc = check_common(&q);
    if (!rc) rc = check_t4_out(q.o, q, q.H, q.Sq);
    if (rc) return rc;
    void* ptr = nullptr;
    if ((rc = noalloc_scratch_ptr(&ptr, reinterpret_cast<hipStream_t>(stream)))) return rc;
    q.kv_workspace = ptr;
  }
  return fwd_stage_impl(&q, SEGPT_FWD_STAGE_PRE, SEGPT_FWD_STAGE_ATTN, stream);
}

int segpt_attn_fwd_stage(const segpt_attn_params* p, int stage, void* stream) {
  if (stage < SEGPT_FWD_STAGE_PRE || stage > SEGPT_FWD_STAGE_ATTN) return SEGPT_E_STAGE;
  return fwd_stage_impl(p, stage, stage, stream);
}

static int bwd_stage_impl(const segpt_attn_params* p_in, int stage_lo, int stage_hi, void* stream) {
  if (!p_in) return SEGPT_E_NULL;
  segpt_attn_params p_copy = *p_in;
  p_copy.flags &= ~SEGPT_FLAG_DECODE;  // a forward-only hint: the backward always works on normalised keys
  const segpt_attn_params* p = &p_copy;
  int rc = check_common(p);
  if (rc) return rc;
  if ((rc = check_bwd(p))) return rc;
  const WsLayout w = bwd_layout(*p);
  KArgs a{};
  a.p = *p;
  char* ws = reinterpret_cast<char*>(p->workspace);
  a.delta = reinterpret_cast<float*>(ws + w.delta);
  a.do_eff = gated_do_copy(*p) ? ws + w.do_eff : nullptr;
  a.dg_part = reinterpret_cast<float*>(ws + w.dg_part);
  a.dcoef_part = reinterpret_cast<float*>(ws + w.dcoef_part);
  if (p->dtype == SEGPT_DTYPE_BF16) {
    a.nlse2 = reinterpret_cast<float*>(ws + w.nlse2);
    a.qhat = reinterpret_cast<uint16_t*>(ws + w.qhat);
  }
  bind_kv(a);
  a.n_dq_blocks = dq_blocks(*p);
  a.n_dkdv_blocks = dkdv_blocks(*p);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool f32 = p->dtype == SEGPT_DTYPE_FP32;
  for (int stage = stage_lo; stage <= stage_hi; ++stage) {
    switch (stage) {
      case SEGPT_BWD_STAGE_PRE:
        rc = f32 ? launch_bwd_pre(a, st) : ((p->flags & SEGPT_FLAG_KV_PREPARED) ? 0 : launch_kv_prep(a, st));
        break;
      case SEGPT_BWD_STAGE_DKDV: rc = f32 ? launch_bwd_dkdv_f32(a, st) : launch_bwd_dkdv_bf16(a, st); break;
      case SEGPT_BWD_STAGE_DQ: rc = f32 ? launch_bwd_dq_f32(a, st) : launch_bwd_dq_bf16(a, st); break;
      case SEGPT_BWD_STAGE_REDUCE: rc = launch_bwd_reduce(a, st); break;
      default: return SEGPT_E_STAGE;
    }
    if (rc) return rc;
  }
  return SEGPT_OK;
}

int segpt_attn_bwd(const segpt_attn_params* p, void* stream) {
  return bwd_stage_impl(p, SEGPT_BWD_STAGE_PRE, SEGPT_BWD_STAGE_REDUCE, stream);
}

int segpt_attn_bwd_stage(const segpt_attn_params* p, int stage, void* stream) {
  if (stage < SEGPT_BWD_STAGE_PRE || stage > SEGPT_BWD_STAGE_REDUCE) return SEGPT_E_STAGE;
  return bwd_stage_impl(p, stage, stage, stream);
}

}  // extern "C"
