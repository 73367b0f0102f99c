// Short causal filter over time on each channel, with the sequence's last inputs in its state slot.
//
//   causal_conv   y_t = sum_j taps[c, j] x_(t - K + 1 + j) (+ bias), optional SiLU, optional + x_t.
//                 Inputs before the portion come from the slot's [K - 1, C] fp32 rows (oldest first),
//                 zeros when the portion starts at position 0 or the sequence has no slot.  An input
//                 bias is added to every row of x on the way in (the slot keeps biased rows).
//   conv_state    the slot takes the last K - 1 inputs after the portion.
//
// One thread per (token, channel); the sum runs in tap order in fp32 whether an input comes from the
// portion or from the slot, so a position's result does not depend on how its prompt was cut.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kActNone = 0, kActSilu = 1;

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
causal_conv_kernel(TO* __restrict__ out, const TI* __restrict__ x, int64_t xs, const float* __restrict__ in_bias,
                   const float* __restrict__ taps, int K, const float* __restrict__ bias, const float* __restrict__ state,
                   const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots,
                   const int* __restrict__ token_seq, int C, int act, int residual) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = token_seq[t];
  const int q0 = cu_q[s];
  const int i = t - q0;
  const int slot = slots[s];
  const bool carry = state != nullptr && slot >= 0 && positions[q0] > 0;
  const float ib = in_bias ? in_bias[c] : 0.f;
  const float* w = taps + static_cast<int64_t>(c) * K;
  float acc = 0.f;
  for (int j = 0; j < K; ++j) {
    const int src = i - (K - 1) + j;
    float v = 0.f;
    if (src >= 0) {
      v = ld<TI>(x + static_cast<int64_t>(q0 + src) * xs + c) + ib;
    } else if (carry) {
      v = state[(static_cast<int64_t>(slot) * (K - 1) + (K - 1 + src)) * C + c];
    }
    acc += w[j] * v;
  }
  if (bias) acc += bias[c];
  if (act == kActSilu) acc = acc * sigmoidf(acc);
  if (residual) acc += ld<TI>(x + static_cast<int64_t>(t) * xs + c) + ib;
  st<TO>(out + static_cast<int64_t>(t) * C + c, acc);
}

// one thread per (sequence, channel): row i of the new state is entry n + i of (old rows, portion rows);
// n >= 1, so every read of an old row lies at or ahead of the row being written
template <typename TI>
__global__ void __launch_bounds__(256)
conv_state_kernel(float* __restrict__ state, const TI* __restrict__ x, int64_t xs, const float* __restrict__ in_bias,
                  const int* __restrict__ cu_q, const int* __restrict__ positions, const int* __restrict__ slots, int K,
                  int C) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int q0 = cu_q[s], n = cu_q[s + 1] - q0, slot = slots[s];
  if (n <= 0 || slot < 0) return;
  const bool carry = positions[q0] > 0;
  const float ib = in_bias ? in_bias[c] : 0.f;
  float* rows = state + static_cast<int64_t>(slot) * (K - 1) * C + c;
  for (int i = 0; i < K - 1; ++i) {
    const int idx = n + i - (K - 1);
    float v = 0.f;
    if (idx >= 0) {
      v = ld<TI>(x + static_cast<int64_t>(q0 + idx) * xs + c) + ib;
    } else if (carry) {
      v = rows[static_cast<int64_t>(n + i) * C];
    }
    rows[static_cast<int64_t>(i) * C] = v;
  }
}

}  // namespace

// x [T, C] rows x_stride elements apart (x_dt); out [T, C] contiguous (out_dt); taps [C, K] fp32; in_bias, bias [C]
// fp32 or null; state [slots, K - 1, C] fp32 (null with K = 1), brought up to date after the outputs
PK_EXPORT int pkm_causal_conv(void* out, int out_dt, const void* x, int x_dt, long long x_stride, const void* in_bias,
                              const void* taps, int K, const void* bias, void* state, const void* cu_q,
                              const void* positions, const void* slots, const void* token_seq, int n_seqs, int T, int C,
                              int act, int residual, hipStream_t stream) {
  if (T <= 0) return 0;
  if (K < 1 || C < 1 || (K > 1 && state == nullptr) || x_stride < C) return -1;
  const dim3 grid(T, (C + 255) / 256);
#define PKM_CC(TI)                                                                                                       \
  PKM_DISPATCH(out_dt, O, causal_conv_kernel<TI, O><<<grid, 256, 0, stream>>>(                                             \
                              static_cast<O*>(out), static_cast<const TI*>(x), x_stride, static_cast<const float*>(in_bias), \
                              static_cast<const float*>(taps), K, static_cast<const float*>(bias),                         \
                              static_cast<const float*>(state), static_cast<const int*>(cu_q),                             \
                              static_cast<const int*>(positions), static_cast<const int*>(slots),                          \
                              static_cast<const int*>(token_seq), C, act, residual))
  if (x_dt == kF32) {
    PKM_CC(float);
  } else if (x_dt == kBF16) {
    PKM_CC(bf16_t);
  } else {
    return -2;
  }
#undef PKM_CC
  int rc = PK_CHECK_LAUNCH();
  if (rc != 0 || K == 1) return rc;
  const dim3 sgrid(n_seqs, (C + 255) / 256);
  PKM_DISPATCH(x_dt, E, conv_state_kernel<E><<<sgrid, 256, 0, stream>>>(
                            static_cast<float*>(state), static_cast<const E*>(x), x_stride, static_cast<const float*>(in_bias),
                            static_cast<const int*>(cu_q), static_cast<const int*>(positions), static_cast<const int*>(slots),
                            K, C));
  return PK_CHECK_LAUNCH();
}
