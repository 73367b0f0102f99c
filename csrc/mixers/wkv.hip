// Time mixing with per-channel data-dependent decays and a matrix state per head.
//
//   shift_mix   mix_n[t] = h[t] + (h[t-1] - h[t]) * mu_n for n mixes at once; the row before a portion's
//               first token is the sequence's slot row (zeros at position 0 or without a slot); a second
//               kernel then leaves the portion's last row in the slot.
//   tanh        in place
//   wkv         per (sequence, head), state S [D, D] fp32 (key channel, value channel):
//                 w_t = exp(-exp(z_t + w0));  o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T
//               A workgroup owns 64 value columns of a (sequence, head); its waves share the key
//               channels of every column's state, kept in registers; r, k, w and u k of a round of 16
//               tokens are staged in LDS (one 16-byte broadcast read per key channel).  Tokens are
//               walked in order with the same order of sums whether a token arrives in a portion or alone.
#include "mix_common.h"

using namespace pkm;

namespace {

template <typename T>
__global__ void __launch_bounds__(256)
shift_mix_kernel(T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu, int n_mix,
                 const float* __restrict__ prev, const int* __restrict__ token_seq, const int* __restrict__ cu_q,
                 const int* __restrict__ positions, const int* __restrict__ slots, int Tn, int W) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int s = token_seq[t];
  const int q0 = cu_q[s];
  const float x = ld<T>(h + static_cast<int64_t>(t) * W + c);
  float p = 0.f;
  if (t > q0) {
    p = ld<T>(h + static_cast<int64_t>(t - 1) * W + c);
  } else {
    const int slot = slots[s];
    if (slot >= 0 && positions[q0] > 0) p = prev[static_cast<int64_t>(slot) * W + c];
  }
  const float d = p - x;
  for (int n = 0; n < n_mix; ++n)
    st<T>(out + (static_cast<int64_t>(n) * Tn + t) * W + c, x + d * mu[static_cast<int64_t>(n) * W + c]);
}

template <typename T>
__global__ void __launch_bounds__(256)
shift_save_kernel(float* __restrict__ prev, const T* __restrict__ h, const int* __restrict__ cu_q,
                  const int* __restrict__ slots, int W) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int last = cu_q[s + 1] - 1, slot = slots[s];
  if (last < cu_q[s] || slot < 0) return;
  prev[static_cast<int64_t>(slot) * W + c] = ld<T>(h + static_cast<int64_t>(last) * W + c);
}

template <typename T>
__global__ void __launch_bounds__(256) tanh_kernel(T* __restrict__ x, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) st<T>(x + i, tanhf(ld<T>(x + i)));
}

constexpr int kRound = 16;  // tokens staged per round

// A workgroup of NW waves owns 64 value columns of a (sequence, head); wave w keeps key channels
// w NR .. w NR + NR - 1 of every column's state in registers (NR NW >= D).  Per round of 16 tokens
// the workgroup stages (r, k, w, u k) of every key channel and v of its columns in LDS with all loads
// issued together, every wave walks the round's tokens over its key channels, and the waves' partial
// outputs are summed in wave order.  grid (column groups of 64, H, sequences).
template <typename T, int NR, int NW>
__global__ void __launch_bounds__(64 * NW)
wkv_kernel(float* __restrict__ out, const T* __restrict__ rkv, int64_t plane, const T* __restrict__ z,
           const float* __restrict__ w0, const float* __restrict__ u, float* __restrict__ state,
           const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots, int H, int D) {
  constexpr int ND = NR * NW, kThreads = 64 * NW;
  __shared__ float4 stage[kRound * ND];       // (r, k, w, u k) per (token of the round, key channel)
  __shared__ float vst[kRound * 64];          // the columns' v per token of the round
  __shared__ float part[NW * kRound * 64];    // the waves' partial outputs
  const int s = blockIdx.z, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int col = blockIdx.x * 64 + lane;
  const int q0 = cu_q[s], q1 = cu_q[s + 1];
  if (q1 <= q0) return;
  const int slot = slots[s];
  const int64_t HD = static_cast<int64_t>(H) * D;
  const bool live = col < D;
  const int d0 = w * NR;
  float S[NR];
  float* sp = slot >= 0 ? state + (static_cast<int64_t>(slot) * H + hd) * D * D + col : nullptr;
  const bool carry = sp != nullptr && positions[q0] > 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) S[i] = (carry && live && d0 + i < D) ? sp[static_cast<int64_t>(d0 + i) * D] : 0.f;
  const T* rp = rkv;
  const T* kp = rkv + plane;
  const T* vp = rkv + 2 * plane;
  const float* w0h = w0 + hd * D;
  const float* uh = u + hd * D;
  constexpr int kPer = kRound * ND / kThreads;  // (token, key channel) pairs per thread and round
  for (int t0 = q0; t0 < q1; t0 += kRound) {
    const int nt = min(kRound, q1 - t0);
    const int n_el = nt * D;
    __syncthreads();
    {
      float rr[kPer], kk[kPer], zz[kPer];
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        const int e = i * kThreads + tid;
        const int j = e / D, d = e - j * D;
        const int64_t at = static_cast<int64_t>(t0 + j) * HD + static_cast<int64_t>(hd) * D + d;
        const bool ok = e < n_el;
        rr[i] = ok ? ld<T>(rp + at) : 0.f;
        kk[i] = ok ? ld<T>(kp + at) : 0.f;
        zz[i] = ok ? ld<T>(z + at) : 0.f;
      }
      float tv[kRound / NW];
#pragma unroll
      for (int i = 0; i < kRound / NW; ++i) {
        const int j = w + i * NW;
        tv[i] = (live && j < nt) ? ld<T>(vp + static_cast<int64_t>(t0 + j) * HD + static_cast<int64_t>(hd) * D + col) : 0.f;
      }
#pragma unroll
      for (int i = 0; i < kPer; ++i) {
        const int e = i * kThreads + tid;
        if (e < n_el) {
          const int j = e / D, d = e - j * D;
          stage[j * ND + d] = float4{rr[i], kk[i], expf(-expf(zz[i] + w0h[d])), uh[d] * kk[i]};
        }
      }
#pragma unroll
      for (int i = 0; i < kRound / NW; ++i) vst[(w + i * NW) * 64 + lane] = tv[i];
    }
    __syncthreads();
    for (int j = 0; j < nt; ++j) {
      const float vv = vst[j * 64 + lane];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        if (d0 + i < D) {
          const float4 f = stage[j * ND + d0 + i];
          o += f.x * (S[i] + f.w * vv);
          S[i] = f.z * S[i] + f.y * vv;
        }
      }
      part[(w * kRound + j) * 64 + lane] = o;
    }
    __syncthreads();
    for (int j = w; j < nt; j += NW) {
      float o = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) o += part[(ww * kRound + j) * 64 + lane];
      if (live) out[static_cast<int64_t>(t0 + j) * HD + static_cast<int64_t>(hd) * D + col] = o;
    }
  }
  if (sp && live) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (d0 + i < D) sp[static_cast<int64_t>(d0 + i) * D] = S[i];
  }
}

}  // namespace

// out [n_mix, T, W]; h [T, W] contiguous; mu [n_mix, W] fp32; prev [slots, W] fp32, updated afterwards
PK_EXPORT int pkm_shift_mix(void* out, const void* h, const void* mu, int n_mix, void* prev, const void* token_seq,
                            const void* cu_q, const void* positions, const void* slots, int n_seqs, int T, int W, int dt,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (n_mix < 1 || W < 1) return -1;
  const dim3 grid(T, (W + 255) / 256);
  PKM_DISPATCH(dt, E, shift_mix_kernel<E><<<grid, 256, 0, stream>>>(
                          static_cast<E*>(out), static_cast<const E*>(h), static_cast<const float*>(mu), n_mix,
                          static_cast<const float*>(prev), static_cast<const int*>(token_seq), static_cast<const int*>(cu_q),
                          static_cast<const int*>(positions), static_cast<const int*>(slots), T, W));
  int rc = PK_CHECK_LAUNCH();
  if (rc != 0) return rc;
  const dim3 sgrid(n_seqs, (W + 255) / 256);
  PKM_DISPATCH(dt, E, shift_save_kernel<E><<<sgrid, 256, 0, stream>>>(static_cast<float*>(prev), static_cast<const E*>(h),
                                                                      static_cast<const int*>(cu_q),
                                                                      static_cast<const int*>(slots), W));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_tanh(void* x, long long n, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  PKM_DISPATCH(dt, E, tanh_kernel<E><<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(static_cast<E*>(x), n));
  return PK_CHECK_LAUNCH();
}

// rkv: r, k, v planes [T, H * D] `plane` elements apart; z [T, H * D]; w0, u [H * D] fp32; state [slots, H, D, D] fp32;
// out [T, H, D] fp32
PK_EXPORT int pkm_wkv(void* out, const void* rkv, long long plane, const void* z, const void* w0, const void* u, void* state,
                      const void* cu_q, const void* positions, const void* slots, int n_seqs, int T, int H, int D, int dt,
                      hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  if (H < 1 || D < 1 || D > 256) return -1;
  const dim3 grid((D + 63) / 64, H, n_seqs);
#define PKM_WKV(NR, NW)                                                                                                 \
  PKM_DISPATCH(dt, E, wkv_kernel<E, NR, NW><<<grid, 64 * NW, 0, stream>>>(                                                 \
                          static_cast<float*>(out), static_cast<const E*>(rkv), plane, static_cast<const E*>(z),           \
                          static_cast<const float*>(w0), static_cast<const float*>(u), static_cast<float*>(state),         \
                          static_cast<const int*>(cu_q), static_cast<const int*>(positions), static_cast<const int*>(slots), \
                          H, D))
  if (D <= 32) {
    PKM_WKV(8, 4);
  } else if (D <= 64) {
    PKM_WKV(16, 4);
  } else if (D <= 128) {
    PKM_WKV(32, 4);
  } else {
    PKM_WKV(32, 8);
  }
#undef PKM_WKV
  return PK_CHECK_LAUNCH();
}
