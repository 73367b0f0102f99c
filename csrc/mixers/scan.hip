// Selective scan: a diagonal state-space recurrence with input-dependent step sizes.
//
//   dt = softplus(d + dt_bias);  S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x_c B_n;
//   y_c = sum_n S[c, n] C_n + D_c x_c;  out_c = y_c * silu(z_c)
//
// A lane owns one channel and keeps its N state numbers and its row of A in registers; a wave owns 64
// channels of a sequence; B and C of a round of tokens are staged in LDS (broadcast reads).  Tokens
// are walked in order with the same order of sums whether a token arrives in a portion or alone.
// State [slots, channels, N] fp32: read by a portion's first token unless it is position 0, written
// after its last token; sequences without a slot start from zeros and leave nothing.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kRound = 16;  // tokens staged per round

__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int NN>
__global__ void __launch_bounds__(64)
selective_scan_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t xs, const T* __restrict__ d, int64_t ds,
                      const float* __restrict__ dt_bias, const float* __restrict__ A, const T* __restrict__ bc, int64_t bcs,
                      const float* __restrict__ skip, const T* __restrict__ z, int64_t zs, float* __restrict__ state,
                      const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots, int C,
                      int N) {
  __shared__ float stage[kRound * 2 * NN];  // B then C of each token of the round
  const int s = blockIdx.y, lane = threadIdx.x;
  const int c = blockIdx.x * 64 + lane;
  const int q0 = cu_q[s], q1 = cu_q[s + 1];
  if (q1 <= q0) return;
  const int slot = slots[s];
  const bool live = c < C;
  float S[NN], a[NN];
  float* sp = (slot >= 0 && live) ? state + (static_cast<int64_t>(slot) * C + c) * N : nullptr;
  const bool carry = sp != nullptr && positions[q0] > 0;
#pragma unroll
  for (int n = 0; n < NN; ++n) {
    S[n] = (carry && n < N) ? sp[n] : 0.f;
    a[n] = (live && n < N) ? A[static_cast<int64_t>(c) * N + n] : 0.f;
  }
  const float db = live ? dt_bias[c] : 0.f, sk = live ? skip[c] : 0.f;
  for (int t0 = q0; t0 < q1; t0 += kRound) {
    const int nt = min(kRound, q1 - t0);
    __syncthreads();
    for (int e = lane; e < nt * 2 * N; e += 64) {
      const int j = e / (2 * N), n = e - j * 2 * N;
      stage[j * 2 * NN + (n < N ? n : NN + n - N)] = ld<T>(bc + static_cast<int64_t>(t0 + j) * bcs + n);
    }
    __syncthreads();
    if (!live) continue;
    for (int j = 0; j < nt; ++j) {
      const int64_t t = t0 + j;
      const float xv = ld<T>(x + t * xs + c);
      const float dt = softplusf(ld<T>(d + t * ds + c) + db);
      const float dx = dt * xv;
      const float* B = stage + j * 2 * NN;
      float y = 0.f;
#pragma unroll
      for (int n = 0; n < NN; ++n) {
        if (n < N) {
          S[n] = expf(dt * a[n]) * S[n] + dx * B[n];
          y += S[n] * B[NN + n];
        }
      }
      y += sk * xv;
      const float zv = ld<T>(z + t * zs + c);
      st<T>(out + t * C + c, y * (zv * sigmoidf(zv)));
    }
  }
  if (sp) {
#pragma unroll
    for (int n = 0; n < NN; ++n)
      if (n < N) sp[n] = S[n];
  }
}

}  // namespace

// x, d, z [T, C] and bc [T, 2N] with their own row strides (all of element type dt); dt_bias, skip [C], A [C, N] fp32;
// state [slots, C, N] fp32; out [T, C] contiguous
PK_EXPORT int pkm_selective_scan(void* out, const void* x, long long xs, const void* d, long long ds, const void* dt_bias,
                                 const void* A, const void* bc, long long bcs, const void* skip, const void* z, long long zs,
                                 void* state, const void* cu_q, const void* positions, const void* slots, int n_seqs, int T,
                                 int C, int N, int dt, hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  if (C < 1 || N < 1 || N > 256) return -1;
  const dim3 grid((C + 63) / 64, n_seqs);
#define PKM_SCAN(NN)                                                                                                      \
  PKM_DISPATCH(dt, E, selective_scan_kernel<E, NN><<<grid, 64, 0, stream>>>(                                                 \
                          static_cast<E*>(out), static_cast<const E*>(x), xs, static_cast<const E*>(d), ds,                   \
                          static_cast<const float*>(dt_bias), static_cast<const float*>(A), static_cast<const E*>(bc), bcs,    \
                          static_cast<const float*>(skip), static_cast<const E*>(z), zs, static_cast<float*>(state),          \
                          static_cast<const int*>(cu_q), static_cast<const int*>(positions), static_cast<const int*>(slots),  \
                          C, N))
  if (N <= 16) {
    PKM_SCAN(16);
  } else if (N <= 32) {
    PKM_SCAN(32);
  } else if (N <= 64) {
    PKM_SCAN(64);
  } else if (N <= 128) {
    PKM_SCAN(128);
  } else {
    PKM_SCAN(256);
  }
#undef PKM_SCAN
  return PK_CHECK_LAUNCH();
}
