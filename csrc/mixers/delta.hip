// Gated delta rule with a short causal filter in front.
//
//   conv_unit    per channel c of the q | k | v projections: y[t] = sum_j taps[c, j] x[t - (K - 1) + j]
//                (inputs before the portion come from the sequence's state slot, zeros at the start
//                of a sequence), SiLU, then every q and k head is set to unit length (q also divided
//                by sqrt(D)); a second kernel brings the slot's last K - 1 inputs up to date
//   delta_rule   per (sequence, head), token by token, S [D, V] fp32:
//                  gate = exp(-exp(A_log_h) softplus(a + dt_bias_h)),  beta = sigmoid(b)
//                  S <- gate S ;  u = beta (v - S^T k) ;  S <- S + k u^T ;  o = S^T q
//
// The state of a (sequence, head) lives in the sequence's state slot between steps.  In delta_rule a
// wave owns 16 value columns; the 4 lanes of a column each hold a quarter of its key rows in
// registers and sum their parts with two lane exchanges, in the same order for every token whether
// it arrives in a long prompt portion or alone.  The first token of a portion reads the slot unless
// it is position 0; the state after the portion's last token is written back.
#include "mix_common.h"

using namespace pkm;

namespace {

__device__ __forceinline__ float siluf(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplusf(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

constexpr int kMaxTaps = 64;  // the kernels loop over the taps; this only bounds a wrong argument

// one wave per (token, head): heads 0..G-1 q, G..2G-1 k, then H value heads
template <typename T>
__global__ void __launch_bounds__(64)
conv_unit_kernel(float* __restrict__ out, const T* __restrict__ proj, int64_t stride, const float* __restrict__ taps, int K,
                 const float* __restrict__ conv_state, const int* __restrict__ cu_q, const int* __restrict__ positions,
                 const int* __restrict__ slots, const int* __restrict__ token_seq, int G, int D, int H, int V) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  const int C = 2 * G * D + H * V;
  const bool qk = item < 2 * G;
  const int width = qk ? D : V;
  const int c0 = qk ? item * D : 2 * G * D + (item - 2 * G) * V;
  const int s = token_seq[t];
  const int a = cu_q[s], slot = slots[s];
  const int i = t - a;  // index inside the portion
  const bool carry = slot >= 0 && positions[a] > 0;
  const float* past = conv_state + static_cast<int64_t>(slot < 0 ? 0 : slot) * (K > 1 ? K - 1 : 1) * C;
  float ss = 0.f;
  for (int d0 = 0; d0 < width; d0 += 64) {
    const int d = d0 + lane;
    float y = 0.f;
    if (d < width) {
      const int c = c0 + d;
      for (int j = 0; j < K; ++j) {
        const int rel = i - (K - 1) + j;
        float x = 0.f;
        if (rel >= 0) {
          x = ld<T>(proj + static_cast<int64_t>(a + rel) * stride + c);
        } else if (carry) {
          x = past[static_cast<int64_t>(K - 1 + rel) * C + c];
        }
        y += taps[static_cast<int64_t>(c) * K + j] * x;
      }
      y = siluf(y);
      ss += y * y;
      out[static_cast<int64_t>(t) * C + c] = y;
    }
  }
  if (!qk) return;
  ss = pk::wave_sum(ss);
  float k = 1.f / sqrtf(ss + 1e-6f);
  if (item < G) k *= 1.f / sqrtf(static_cast<float>(D));
  for (int d = lane; d < width; d += 64) out[static_cast<int64_t>(t) * C + c0 + d] *= k;  // the lane's own values
}

// new state[j] = the input K - 1 - j steps before the portion's end; thread per (sequence, channel)
template <typename T>
__global__ void __launch_bounds__(256)
conv_state_kernel(float* __restrict__ conv_state, const T* __restrict__ proj, int64_t stride, int K,
                  const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots, int C) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int a = cu_q[s], n = cu_q[s + 1] - a, slot = slots[s];
  if (slot < 0 || n <= 0) return;
  const bool carry = positions[a] > 0;
  float* st_ = conv_state + static_cast<int64_t>(slot) * (K - 1) * C;
  for (int j = 0; j < K - 1; ++j) {  // ascending: a read of old[j + n] comes before any write at or above it
    const int rel = n - (K - 1) + j;
    float x = 0.f;
    if (rel >= 0) {
      x = ld<T>(proj + static_cast<int64_t>(a + rel) * stride + c);
    } else if (carry) {
      x = st_[static_cast<int64_t>(K - 1 + rel) * C + c];
    }
    st_[static_cast<int64_t>(j) * C + c] = x;
  }
}

constexpr int kMaxChunk = 16;  // tokens staged per group (fewer when a head is wide)
constexpr int kCols = 64;      // value columns per workgroup (4 waves x 16)

// sums over the 4 lanes of a quad (data-parallel lane exchanges inside the quad)
__device__ __forceinline__ float quad_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
  return v;
}

// AT: element type of the a | b pre-activations.  Lane `sub` of a column's quad keeps key rows
// sub * nd .. sub * nd + nd - 1 (nd = ceil(D / 4) <= ND; rows past D hold zeros) in registers; q and
// k of a token lie in LDS as 4 runs of ND (+ 4 floats of padding, so the quad's four 16-byte reads
// fall on different banks).  The next group's q, k, v are fetched into registers before the
// current group is computed.
template <typename AT, int ND>
__global__ void __launch_bounds__(256)
delta_rule_kernel(float* __restrict__ out, const float* __restrict__ qkv, const AT* __restrict__ ab, int64_t ab_stride,
                  const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
                  const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots, int G, int D,
                  int H, int V, int kChunk) {
  constexpr int RS = ND + 4, TS = 4 * RS;          // floats per run and per token
  constexpr int QK_IT = (kMaxChunk * 4 * ND + 255) / 256, V_IT = (kMaxChunk * kCols + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* qs = smem;                 // [kChunk][4][RS]
  float* ks = qs + kChunk * TS;     // [kChunk][4][RS]
  float* vs = ks + kChunk * TS;     // [kChunk][kCols]
  float* gs = vs + kChunk * kCols;  // [kChunk] gate
  float* bs_ = gs + kChunk;         // [kChunk] beta
  const int s = blockIdx.x / H, h = blockIdx.x - s * H;
  const int v0 = blockIdx.y * kCols;
  const int a = cu_q[s], b = cu_q[s + 1];
  if (b <= a) return;
  const int tid = threadIdx.x, sub = tid & 3, col = v0 + (tid >> 2);
  const int slot = slots[s];
  const int C = 2 * G * D + H * V;
  const int nd = (D + 3) / 4;
  const int kvh = h / (H / G);
  const float neg_rate = -expf(a_log[h]), bias = dt_bias[h];
  float* sp = slot >= 0 ? state + ((static_cast<int64_t>(slot) * H + h) * D) * V : nullptr;
  const bool carry = sp != nullptr && positions[a] > 0;
  float S[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = sub * nd + i;
    S[i] = (carry && i < nd && d < D && col < V) ? sp[static_cast<int64_t>(d) * V + col] : 0.f;
  }
  const int64_t qo = static_cast<int64_t>(kvh) * D, ko = static_cast<int64_t>(G + kvh) * D;
  const int64_t vo = 2 * static_cast<int64_t>(G) * D + static_cast<int64_t>(h) * V + v0;
  float rq[QK_IT], rk[QK_IT], rv[V_IT];
  auto fetch = [&](int t0) {  // the group starting at token t0 (zeros outside the head's D rows)
    const int nt = min(kChunk, b - t0);
#pragma unroll
    for (int i = 0; i < QK_IT; ++i) {
      const int e = tid + 256 * i, t = e / (4 * ND), r = e - t * 4 * ND, su = r / ND, ii = r - su * ND;
      const int d = su * nd + ii;
      const bool ok = t < nt && ii < nd && d < D;
      const float* row = qkv + static_cast<int64_t>(t0 + (ok ? t : 0)) * C;
      rq[i] = ok ? row[qo + d] : 0.f;
      rk[i] = ok ? row[ko + d] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < V_IT; ++i) {
      const int e = tid + 256 * i, t = e / kCols, c = e - t * kCols;
      const bool ok = t < nt && v0 + c < V;
      rv[i] = ok ? qkv[static_cast<int64_t>(t0 + t) * C + vo + c] : 0.f;
    }
  };
  fetch(a);
  for (int t0 = a; t0 < b; t0 += kChunk) {
    const int nt = min(kChunk, b - t0);
    __syncthreads();  // the group before has been read
#pragma unroll
    for (int i = 0; i < QK_IT; ++i) {
      const int e = tid + 256 * i, t = e / (4 * ND), r = e - t * 4 * ND, su = r / ND, ii = r - su * ND;
      if (t < kChunk) {
        qs[t * TS + su * RS + ii] = rq[i];
        ks[t * TS + su * RS + ii] = rk[i];
      }
    }
#pragma unroll
    for (int i = 0; i < V_IT; ++i) {
      const int e = tid + 256 * i;
      if (e < kChunk * kCols) vs[e] = rv[i];
    }
    if (tid < nt) {
      const AT* r = ab + static_cast<int64_t>(t0 + tid) * ab_stride;
      gs[tid] = expf(neg_rate * softplusf(ld<AT>(r + h) + bias));
      bs_[tid] = sigmoidf(ld<AT>(r + H + h));
    }
    __syncthreads();
    if (t0 + kChunk < b) fetch(t0 + kChunk);  // in flight while this group is computed
    for (int t = 0; t < nt; ++t) {
      const float gate = gs[t], beta = bs_[t];
      const float vv = vs[t * kCols + (tid >> 2)];
      const float4* kr = reinterpret_cast<const float4*>(ks + t * TS + sub * RS);
      const float4* qr = reinterpret_cast<const float4*>(qs + t * TS + sub * RS);
      float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
#pragma unroll
      for (int i = 0; i < ND / 4; ++i) {
        const float4 k4 = kr[i];
        r0 += S[4 * i] * k4.x;
        r1 += S[4 * i + 1] * k4.y;
        r2 += S[4 * i + 2] * k4.z;
        r3 += S[4 * i + 3] * k4.w;
      }
      const float r = gate * quad_sum((r0 + r1) + (r2 + r3));  // (gate S)^T k
      const float u = beta * (vv - r);
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int i = 0; i < ND / 4; ++i) {
        const float4 k4 = kr[i], q4 = qr[i];
        S[4 * i] = gate * S[4 * i] + k4.x * u;
        o0 += S[4 * i] * q4.x;
        S[4 * i + 1] = gate * S[4 * i + 1] + k4.y * u;
        o1 += S[4 * i + 1] * q4.y;
        S[4 * i + 2] = gate * S[4 * i + 2] + k4.z * u;
        o2 += S[4 * i + 2] * q4.z;
        S[4 * i + 3] = gate * S[4 * i + 3] + k4.w * u;
        o3 += S[4 * i + 3] * q4.w;
      }
      const float o = quad_sum((o0 + o1) + (o2 + o3));
      if (sub == 0 && col < V) out[(static_cast<int64_t>(t0 + t) * H + h) * V + col] = o;
    }
  }
  if (sp != nullptr && col < V) {
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = sub * nd + i;
      if (i < nd && d < D) sp[static_cast<int64_t>(d) * V + col] = S[i];
    }
  }
}

}  // namespace

// out fp32 [T, C], C = 2 G D + H V; proj [T, C] rows `stride` elements apart; taps [C, K] fp32;
// conv_state [slots, K - 1, C] fp32 (read, then brought up to date by a second launch)
PK_EXPORT int pkm_conv_unit(void* out, const void* proj, long long stride, const void* taps, int K, void* conv_state,
                            const void* cu_q, const void* positions, const void* slots, const void* token_seq, int n_seqs,
                            int T, int G, int D, int H, int V, int dt, hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  if (K < 1 || K > kMaxTaps || G < 1 || H < 1 || D < 1 || V < 1) return -1;
  const int C = 2 * G * D + H * V;
  const dim3 grid(T, 2 * G + H);
  PKM_DISPATCH(dt, E, conv_unit_kernel<E><<<grid, 64, 0, stream>>>(
                          static_cast<float*>(out), static_cast<const E*>(proj), stride, static_cast<const float*>(taps), K,
                          static_cast<const float*>(conv_state), static_cast<const int*>(cu_q),
                          static_cast<const int*>(positions), static_cast<const int*>(slots),
                          static_cast<const int*>(token_seq), G, D, H, V));
  int rc = PK_CHECK_LAUNCH();
  if (rc || K == 1) return rc;
  const dim3 sgrid((C + 255) / 256, n_seqs);
  PKM_DISPATCH(dt, E, conv_state_kernel<E><<<sgrid, 256, 0, stream>>>(
                          static_cast<float*>(conv_state), static_cast<const E*>(proj), stride, K,
                          static_cast<const int*>(cu_q), static_cast<const int*>(positions), static_cast<const int*>(slots),
                          C));
  return PK_CHECK_LAUNCH();
}

// out [T, H, V] fp32; qkv fp32 [T, G*D | G*D | H*V]; ab [T, H | H] rows ab_stride elements apart
// (ab_dt); state [slots, H, D, V] fp32
PK_EXPORT int pkm_delta_rule(void* out, const void* qkv, const void* ab, long long ab_stride, int ab_dt, const void* a_log,
                             const void* dt_bias, void* state, const void* cu_q, const void* positions, const void* slots,
                             int n_seqs, int T, int G, int D, int H, int V, hipStream_t stream) {
  if (n_seqs <= 0 || T <= 0) return 0;
  if (D < 1 || D > 512 || V < 1 || G < 1 || H % G) return -1;
  const dim3 grid(n_seqs * H, (V + kCols - 1) / kCols);
  const int nd = (D + 3) / 4;
  const int ndt = nd <= 8 ? 8 : nd <= 16 ? 16 : nd <= 32 ? 32 : nd <= 64 ? 64 : 128;
  const int per_tok = 8 * (ndt + 4) + kCols + 2;  // floats of LDS per staged token
  const int chunk = max(1, min(kMaxChunk, 15360 / per_tok));  // at most 60 KiB of LDS
  const size_t lds = static_cast<size_t>(chunk) * per_tok * sizeof(float);
#define PKM_DELTA(ND)                                                                                                 \
  PKM_DISPATCH(ab_dt, E, delta_rule_kernel<E, ND><<<grid, 256, lds, stream>>>(                                          \
                             static_cast<float*>(out), static_cast<const float*>(qkv), static_cast<const E*>(ab), ab_stride, \
                             static_cast<const float*>(a_log), static_cast<const float*>(dt_bias),                     \
                             static_cast<float*>(state), static_cast<const int*>(cu_q), static_cast<const int*>(positions), \
                             static_cast<const int*>(slots), G, D, H, V, chunk))
  if (nd <= 8) {
    PKM_DELTA(8);
  } else if (nd <= 16) {
    PKM_DELTA(16);
  } else if (nd <= 32) {
    PKM_DELTA(32);
  } else if (nd <= 64) {
    PKM_DELTA(64);
  } else {
    PKM_DELTA(128);
  }
#undef PKM_DELTA
  return PK_CHECK_LAUNCH();
}
