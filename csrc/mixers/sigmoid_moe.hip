// Mixture of experts with sigmoid scores that scale the expert's INPUT.
//
//   route_sigmoid_topk   z = W_r x in fp32 (x: the fp32 residual row), s = sigmoid(z); the `top`
//                        largest s and their experts (ties: the lower expert), not renormalised
//   expert_gate_up       rows sorted by expert (offsets / sorted slots from the expert align
//                        kernel): h[r] = silu(s_r * (W_gate[e] x_t)) * (s_r * (W_up[e] x_t))
//                        -- the score applied to the two products, which equals scaling the input
//                        and keeps the products' fp32 accumulations unscaled
//   expert_down          y[r] = W_down[e] h[r], fp32 out
//   combine_rows         out[t] = sum over the token's `top` slots of y[inv[slot]]   (plain sum)
//
// The grouped products tile each expert's rows by 32: a workgroup finds its expert from the
// device-side offsets (no host read-back), an expert without rows costs nothing.  FMA tiles in
// fp32 for both element types.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kMaxTop = 16;

// One wave per token.  WITH_DOT: the logits are computed here, z[e] = x . wr[e] (small batches:
// one launch, a fixed summation order).  Otherwise `x` holds the fp32 logits [T, E] of a library
// fp32 GEMM (large batches).  Then s = sigmoid(z) and `top` rounds of arg-max over the experts.
template <bool WITH_DOT>
__global__ void __launch_bounds__(64)
route_sigmoid_topk_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ x,
                          const float* __restrict__ wr, int W, int E, int top) {
  extern __shared__ float sc[];  // [E]
  const int t = blockIdx.x, lane = threadIdx.x;
  if (WITH_DOT) {
    const float* xr = x + static_cast<int64_t>(t) * W;
    for (int e = 0; e < E; ++e) {
      const float* w = wr + static_cast<int64_t>(e) * W;
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
      int i = lane;
      for (; i + 192 < W; i += 256) {  // four independent loads in flight per lane
        d0 += xr[i] * w[i];
        d1 += xr[i + 64] * w[i + 64];
        d2 += xr[i + 128] * w[i + 128];
        d3 += xr[i + 192] * w[i + 192];
      }
      for (; i < W; i += 64) d0 += xr[i] * w[i];
      const float d = pk::wave_sum((d0 + d1) + (d2 + d3));
      if (lane == 0) sc[e] = sigmoidf(d);
    }
  } else {
    for (int e = lane; e < E; e += 64) sc[e] = sigmoidf(x[static_cast<int64_t>(t) * E + e]);
  }
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    float best = -1.f;
    int bi = E;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > best) {  // ascending e per lane: the first of equal scores stays
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) {
        best = ov;
        bi = oi;
      }
    }
    if (lane == 0) {
      ids[t * top + k] = bi;
      wts[t * top + k] = best;
      sc[bi] = -2.f;
    }
    __syncthreads();
  }
}

constexpr int kBM = 32, kBN = 32, kBK = 32;

// which expert and row range does m-tile `tile` cover; false: past the last tile
__device__ __forceinline__ bool find_tile(const int* offsets, int E, int tile, int& e, int& r0, int& r1) {
  for (e = 0; e < E; ++e) {
    const int lo = offsets[e], hi = offsets[e + 1];
    const int nt = (hi - lo + kBM - 1) / kBM;
    if (tile < nt) {
      r0 = lo + tile * kBM;
      r1 = min(hi, r0 + kBM);
      return true;
    }
    tile -= nt;
  }
  return false;
}

// C[r, n] = sum_k A[arow(r), k] * B[e][n, k]   (B: [E, N, K]); DUAL: a second B and a gated
// epilogue: with slot_scale the scaled SiLU product, without it the clamped product
// min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u, -limit, limit) + 1), or with limit <= 0 the plain
// SiLU product silu(g) * u.  256 threads: thread (ty, tx) owns rows ty, ty + 16 and columns tx, tx + 16.
template <typename T, typename TA, typename TC, bool DUAL>
__global__ void __launch_bounds__(256)
grouped_rows_kernel(TC* __restrict__ C, const TA* __restrict__ A, const T* __restrict__ B0, const T* __restrict__ B1,
                    const int* __restrict__ offsets, const int* __restrict__ sorted_slots,
                    const float* __restrict__ slot_scale, int top, int E, int N, int K, float limit) {
  __shared__ float as[kBM][kBK + 1];
  __shared__ float b0s[kBN][kBK + 1];
  __shared__ float b1s[DUAL ? kBN : 1][kBK + 1];
  int e, r0, r1;
  if (!find_tile(offsets, E, blockIdx.x, e, r0, r1)) return;
  const int n0 = blockIdx.y * kBN;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const T* b0 = B0 + static_cast<int64_t>(e) * N * K;
  const T* b1 = DUAL ? B1 + static_cast<int64_t>(e) * N * K : nullptr;
  float acc0[2][2] = {{0.f, 0.f}, {0.f, 0.f}}, acc1[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  for (int k0 = 0; k0 < K; k0 += kBK) {
    for (int i = tid; i < kBM * kBK; i += 256) {
      const int r = i / kBK, c = i - r * kBK;
      float v = 0.f;
      if (r0 + r < r1 && k0 + c < K) {
        const int64_t arow = sorted_slots ? sorted_slots[r0 + r] / top : r0 + r;
        v = ld<TA>(A + arow * K + k0 + c);
      }
      as[r][c] = v;
    }
    for (int i = tid; i < kBN * kBK; i += 256) {
      const int r = i / kBK, c = i - r * kBK;
      const bool ok = n0 + r < N && k0 + c < K;
      b0s[r][c] = ok ? ld<T>(b0 + static_cast<int64_t>(n0 + r) * K + k0 + c) : 0.f;
      if (DUAL) b1s[r][c] = ok ? ld<T>(b1 + static_cast<int64_t>(n0 + r) * K + k0 + c) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int c = 0; c < kBK; ++c) {
      const float a0 = as[ty][c], a1 = as[ty + 16][c];
      const float w0 = b0s[tx][c], w1 = b0s[tx + 16][c];
      acc0[0][0] += a0 * w0;
      acc0[0][1] += a0 * w1;
      acc0[1][0] += a1 * w0;
      acc0[1][1] += a1 * w1;
      if (DUAL) {
        const float u0 = b1s[tx][c], u1 = b1s[tx + 16][c];
        acc1[0][0] += a0 * u0;
        acc1[0][1] += a0 * u1;
        acc1[1][0] += a1 * u0;
        acc1[1][1] += a1 * u1;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = r0 + ty + 16 * i;
    if (r >= r1) continue;
    const float s = (DUAL && slot_scale) ? slot_scale[sorted_slots[r]] : 1.f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      float v = acc0[i][j];
      if (DUAL && slot_scale) {
        const float g = s * v, u = s * acc1[i][j];
        v = g * sigmoidf(g) * u;
      } else if (DUAL && limit > 0.f) {
        const float g = fminf(v, limit), u = fminf(fmaxf(acc1[i][j], -limit), limit);
        v = g * sigmoidf(1.702f * g) * (u + 1.f);
      } else if (DUAL) {
        v = v * sigmoidf(v) * acc1[i][j];
      }
      st<TC>(C + static_cast<int64_t>(r) * N + n, v);
    }
  }
}

// Expert align for more experts than the 64 of the stable single-wave sort: offsets [E + 1],
// sorted slots, inverse positions.  One workgroup; rows of one expert land in arrival order of
// the LDS atomics, which no result depends on (every grouped row is computed on its own).
__global__ void __launch_bounds__(1024) expert_align_wide_kernel(const int* __restrict__ ids, int n, int E,
                                                                 int* __restrict__ offsets, int* __restrict__ sorted,
                                                                 int* __restrict__ inv) {
  extern __shared__ int cnt[];  // [E] counts, then [E] cursors
  int* cur = cnt + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = run;
      cur[e] = run;
      run += cnt[e];
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int at = atomicAdd(&cur[ids[i]], 1);
    sorted[at] = i;
    inv[i] = at;
  }
}

template <typename Y>
__global__ void __launch_bounds__(256) combine_rows_kernel(float* __restrict__ out, const Y* __restrict__ y,
                                                           const int* __restrict__ inv, int top, int W) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float a = 0.f;
    for (int k = 0; k < top; ++k) {
      const int r = inv[t * top + k];
      if (r >= 0) a += ld<Y>(y + static_cast<int64_t>(r) * W + i);
    }
    out[static_cast<int64_t>(t) * W + i] = a;
  }
}

// rows in expert order, each the fp32 stream row of its token times the slot's score: the input
// of the framework's grouped expert GEMMs (the score scales the expert's input)
template <typename T>
__global__ void __launch_bounds__(256) permute_scaled_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                             const int* __restrict__ sorted_slots,
                                                             const float* __restrict__ slot_scale, int top, int W) {
  const int r = blockIdx.x;
  const int slot = sorted_slots[r];
  const float s = slot_scale[slot];
  const float* src = x + static_cast<int64_t>(slot / top) * W;
  T* dst = out + static_cast<int64_t>(r) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) st<T>(dst + i, s * src[i]);
}

}  // namespace

PK_EXPORT int pkm_route_sigmoid_topk(void* ids, void* wts, const void* x, const void* wr, int T, int W, int E, int top,
                                     hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || top > E || top > kMaxTop || E > 4096) return -1;
  // wr == nullptr: x holds the logits [T, E]
  if (wr)
    route_sigmoid_topk_kernel<true><<<T, 64, E * sizeof(float), stream>>>(
        static_cast<int*>(ids), static_cast<float*>(wts), static_cast<const float*>(x), static_cast<const float*>(wr), W,
        E, top);
  else
    route_sigmoid_topk_kernel<false><<<T, 64, E * sizeof(float), stream>>>(
        static_cast<int*>(ids), static_cast<float*>(wts), static_cast<const float*>(x), nullptr, W, E, top);
  return PK_CHECK_LAUNCH();
}

// h [n_rows, F] (element type dt) from x [T, W], gate / up [E, F, W]
PK_EXPORT int pkm_expert_gate_up(void* h, const void* x, const void* gate, const void* up, const void* offsets,
                                 const void* sorted_slots, const void* slot_scale, int n_rows, int top, int E, int F,
                                 int W, int dt, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const dim3 grid((n_rows + kBM - 1) / kBM + E, (F + kBN - 1) / kBN);
  PKM_DISPATCH(dt, T, grouped_rows_kernel<T, T, T, true><<<grid, 256, 0, stream>>>(
                          static_cast<T*>(h), static_cast<const T*>(x), static_cast<const T*>(gate),
                          static_cast<const T*>(up), static_cast<const int*>(offsets),
                          static_cast<const int*>(sorted_slots), static_cast<const float*>(slot_scale), top, E, F, W,
                          0.f));
  return PK_CHECK_LAUNCH();
}

// the same with the clamped epilogue (no scores): h = min(g, limit) sigmoid(1.702 min(g, limit)) (clamp(u) + 1);
// limit <= 0: h = silu(g) u
PK_EXPORT int pkm_expert_gate_up_clamped(void* h, const void* x, const void* gate, const void* up, const void* offsets,
                                         const void* sorted_slots, float limit, int n_rows, int top, int E, int F,
                                         int W, int dt, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const dim3 grid((n_rows + kBM - 1) / kBM + E, (F + kBN - 1) / kBN);
  PKM_DISPATCH(dt, T, grouped_rows_kernel<T, T, T, true><<<grid, 256, 0, stream>>>(
                          static_cast<T*>(h), static_cast<const T*>(x), static_cast<const T*>(gate),
                          static_cast<const T*>(up), static_cast<const int*>(offsets),
                          static_cast<const int*>(sorted_slots), nullptr, top, E, F, W, limit));
  return PK_CHECK_LAUNCH();
}

// y [n_rows, W] fp32 from h [n_rows, F], down [E, W, F]
PK_EXPORT int pkm_expert_down(void* y, const void* h, const void* down, const void* offsets, int n_rows, int E, int W,
                              int F, int dt, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const dim3 grid((n_rows + kBM - 1) / kBM + E, (W + kBN - 1) / kBN);
  PKM_DISPATCH(dt, T, grouped_rows_kernel<T, T, float, false><<<grid, 256, 0, stream>>>(
                          static_cast<float*>(y), static_cast<const T*>(h), static_cast<const T*>(down), nullptr,
                          static_cast<const int*>(offsets), nullptr, nullptr, 1, E, W, F, 0.f));
  return PK_CHECK_LAUNCH();
}

// y_dt: element type of the expert outputs y
PK_EXPORT int pkm_combine_rows(void* out, const void* y, const void* inv, int T, int top, int W, int y_dt,
                               hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(y_dt, Y, combine_rows_kernel<Y><<<T, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const Y*>(y),
                                                                      static_cast<const int*>(inv), top, W));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_permute_scaled(void* out, const void* x, const void* sorted_slots, const void* slot_scale, int n,
                                 int top, int W, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  PKM_DISPATCH(dt, T, permute_scaled_kernel<T><<<n, 256, 0, stream>>>(
                          static_cast<T*>(out), static_cast<const float*>(x), static_cast<const int*>(sorted_slots),
                          static_cast<const float*>(slot_scale), top, W));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_expert_align_wide(const void* ids, void* offsets, void* sorted, void* inv, int n, int E,
                                    hipStream_t stream) {
  if (E < 1 || E > 4096) return -1;
  expert_align_wide_kernel<<<1, 1024, 2 * E * sizeof(int), stream>>>(static_cast<const int*>(ids), n, E,
                                                                     static_cast<int*>(offsets),
                                                                     static_cast<int*>(sorted), static_cast<int*>(inv));
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_abi_version() { return 1; }
