// Microbenchmark behind one structural decision of this library: why the backward is two deterministic kernels (seven
// matrix products) and not one key-stationary kernel in the shape of the reference's
// (triton_flash_attn_qknorm.py:192-255, dQ by tl.atomic_add at :229; five products).
//
// It issues exactly the dQ traffic such a kernel would generate at the IMU-1 shape (B=8, 18 query / 6 kv heads,
// S=2048, head_dim 64, causal) and nothing else: every (batch, kv head, key tile) workgroup adds, for every visible
// 64-query tile of its 3 query heads, a 64x64 fp32 tile into a [B,H,S,D] accumulator.
//   mode 0  global_atomic_add_f32 (no return value)
//   mode 1  plain stores to the same addresses (what the memory system can take)
//   mode 2  load + add + store (racy: traffic only)
//   mode 3  global_atomic_pk_add_bf16 into a bf16 accumulator (half the payload, bf16 accumulation)
// with 128 or 256 keys per workgroup, with and without pinning a (batch, kv head) pair to one XCD.
// Build: python -m sample_efficient_gpt_amd.build   (writes sample_efficient_gpt_amd/dq_atomic_floor.bin)
// Run:   sample_efficient_gpt_amd/dq_atomic_floor.bin
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("hip error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)

// grid: pairs * n_kt workgroups, 256 threads; MODE 0: atomic add, 1: plain store (same addresses), 2: load+add+store (racy, traffic only)
template <int MODE>
__global__ __launch_bounds__(256, 2) void atom_kernel(float* dq, int B, int H, int Hkv, int S, int keys_per_wg, int xcd_pin) {
  const int D = 64;
  const int rep = H / Hkv;
  const int n_kt = S / keys_per_wg;
  const int pairs = B * Hkv;
  int bid = blockIdx.x;
  int pair, kt;
  if (xcd_pin) {
    const int xcd = bid & 7, slot = bid >> 3, pp = pairs >> 3;
    const int trev = slot / pp;
    pair = (slot - trev * pp) * 8 + xcd;
    kt = trev;  // early key tiles first (heaviest)
  } else {
    pair = bid % pairs; kt = bid / pairs;
  }
  const int b = pair / Hkv, g = pair % Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, hh = lane >> 5;
  const int qb = wave >> 1, mb = wave & 1;
  const int qt0 = kt * keys_per_wg / 64;
  const int n_qt = S / 64;
  float v = 1.0f;
  for (int hq = 0; hq < rep; ++hq) {
    const int h = g * rep + hq;
    float* base = dq + ((size_t)(b * H + h) * S) * D;
    for (int t = qt0; t < n_qt; ++t) {
      float* p = base + (size_t)(t * 64 + 32 * qb) * D + 32 * mb + ln;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * hh + (r & 3);
        if (MODE == 0) atomicAdd(p + row * D, v);   // no return value used -> global_atomic_add_f32
        else if (MODE == 1) __builtin_nontemporal_store(v, p + row * D);
        else if (MODE == 2) p[row * D] += v;
        else if (mb == 0) {  // bf16 accumulator [.., D] bf16: lane ln adds the column pair (2 ln, 2 ln + 1) of the row
          typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
          typedef bf2 __attribute__((address_space(1))) * gbf2_ptr;
          const bf2 one = {(__bf16)1.0f, (__bf16)1.0f};
          __bf16* acc = reinterpret_cast<__bf16*>(base) + (size_t)(t * 64 + 32 * qb + row) * D + 2 * ln;
          __builtin_amdgcn_global_atomic_fadd_v2bf16((gbf2_ptr)acc, one);
        }
      }
    }
  }
}

int main(int argc, char** argv) {
  const int B = 8, H = 18, Hkv = 6, S = 2048, D = 64;
  const size_t n = (size_t)B * H * S * D;
  float* dq;
  CK(hipMalloc(&dq, n * 4));
  CK(hipMemset(dq, 0, n * 4));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (int kpw : {128, 256}) {
    for (int pin = 0; pin < 2; ++pin) {
      for (int mode = 0; mode < 4; ++mode) {
        const int grid = B * Hkv * (S / kpw);
        float best = 1e9f;
        for (int it = 0; it < 6; ++it) {
          CK(hipEventRecord(e0));
          if (mode == 0) hipLaunchKernelGGL(atom_kernel<0>, dim3(grid), dim3(256), 0, 0, dq, B, H, Hkv, S, kpw, pin);
          if (mode == 1) hipLaunchKernelGGL(atom_kernel<1>, dim3(grid), dim3(256), 0, 0, dq, B, H, Hkv, S, kpw, pin);
          if (mode == 2) hipLaunchKernelGGL(atom_kernel<2>, dim3(grid), dim3(256), 0, 0, dq, B, H, Hkv, S, kpw, pin);
          if (mode == 3) hipLaunchKernelGGL(atom_kernel<3>, dim3(grid), dim3(256), 0, 0, dq, B, H, Hkv, S, kpw, pin);
          CK(hipEventRecord(e1));
          CK(hipEventSynchronize(e1));
          float ms; CK(hipEventElapsedTime(&ms, e0, e1));
          if (it > 0 && ms < best) best = ms;
        }
        // bytes of atomic payload
        double tiles = 0; for (int kt = 0; kt < S / kpw; ++kt) tiles += (S / 64 - kt * kpw / 64);
        double bytes = tiles * B * H * 64.0 * 64 * (mode == 3 ? 2 : 4);
        printf("keys/wg %d pin %d mode %d: %.1f us  payload %.0f MB  %.2f TB/s\n", kpw, pin, mode, best * 1e3, bytes / 1e6, bytes / best / 1e9);
        fflush(stdout);
      }
    }
  }
  CK(hipFree(dq));
  return 0;
}
