// Residual streams of pre-norm layers, kept in fp32, one or several per token (hyper-connections).
//
//   spread_rows   xs[t, s] = table[ids[t]] * scale for every stream s
//   hyper_step    closes one sublayer and opens the next, per token, in one pass:
//                   y      = the sublayer's output row: a plain row, the sum of split-K slabs, or a
//                            mixture's  sum_j wts[t, j] * rows[inv[t, j]]  (+ [sigmoid(gate[t]) *] shared[t])
//                   xs'[t] = sum_s mix[s, t] xs[s] + a_out[t] y          (all streams from the old ones)
//                   u      = sum_t a_in[t] xs'[t];  z = u / sqrt(mean(u^2) + eps) * w
//                 either half may be absent; with `rows` only those tokens are opened (the rows whose
//                 logits are wanted).  S = 1 with unit coefficients is the plain residual.
//   tanh_cap      x <- cap * tanh(x / cap)
//
// One workgroup per token; every sum runs in a fixed order, so a token's result does not depend
// on the rest of the batch.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kMaxStreams = 8;

template <typename T>
__global__ void __launch_bounds__(256) spread_rows_kernel(float* __restrict__ xs, const T* __restrict__ table,
                                                          const int* __restrict__ ids, int S, int W, int vocab,
                                                          float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + static_cast<int64_t>(id) * W;
  float* dst = xs + static_cast<int64_t>(t) * S * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = ld<T>(src + i) * scale;
    for (int s = 0; s < S; ++s) dst[s * W + i] = v;
  }
}

struct HyperArgs {
  float* xs;
  int S, W;
  const void* y;
  int nslab;
  int64_t slab_stride;
  const int* inv;
  int top;
  const float* wts;
  const void* y2;
  const float* g2;
  int64_t g2_stride;
  const float* mix;
  const float* a_out;
  const float* a_in;
  const float* norm_w;
  float eps;
  void* act;
  float* z32;
  const int* rows;
};

// four consecutive coordinates per thread (W % 4 == 0): 16-byte loads of the fp32 streams
template <typename E>
__device__ __forceinline__ float4 ld4(const E* p);
template <>
__device__ __forceinline__ float4 ld4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <>
__device__ __forceinline__ float4 ld4<bf16_t>(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                __uint_as_float(v.y & 0xffff0000u)};
}
template <typename E>
__device__ __forceinline__ void st4(E* p, float4 v);
template <>
__device__ __forceinline__ void st4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <>
__device__ __forceinline__ void st4<bf16_t>(bf16_t* p, float4 v) {
  uint2 w;
  w.x = pk::pack2(v.x, v.y);
  w.y = pk::pack2(v.z, v.w);
  *reinterpret_cast<uint2*>(p) = w;
}
__device__ __forceinline__ float4 fma4(float c, float4 a, float4 b) {
  return float4{c * a.x + b.x, c * a.y + b.y, c * a.z + b.z, c * a.w + b.w};
}

// VEC >= 4 (= 4 * groups per thread): W % 4 == 0, every thread owns up to VEC / 4 groups of four
// consecutive coordinates and keeps the opened sum in registers between the two passes; VEC = 1: any
// W, one coordinate at a time, the opened sum in LDS
template <typename T, typename Y, int VEC>
__global__ void __launch_bounds__(1024) hyper_step_kernel(HyperArgs a) {
  constexpr int NG = VEC >= 4 ? VEC / 4 : 1;
  __shared__ float red[16];
  __shared__ float cf[kMaxStreams * kMaxStreams + 2 * kMaxStreams];
  extern __shared__ __attribute__((aligned(16))) float vbuf[];  // [W] the opened sum u, kept between the two passes
  const int r = blockIdx.x;
  const int S = a.S, W = a.W;
  const int64_t src = a.rows ? a.rows[r] : r;
  float* x = a.xs + src * S * W;
  const bool close = a.mix != nullptr, open = a.a_in != nullptr;
  float* c_mix = cf;
  float* c_out = cf + kMaxStreams * kMaxStreams;
  float* c_in = c_out + kMaxStreams;
  if (threadIdx.x < S * S && close) c_mix[threadIdx.x] = a.mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (close) c_out[threadIdx.x] = a.a_out[threadIdx.x];
    if (open) c_in[threadIdx.x] = a.a_in[threadIdx.x];
  }
  __syncthreads();
  const Y* y = static_cast<const Y*>(a.y);
  const T* y2 = static_cast<const T*>(a.y2);
  const float gate = y2 ? (a.g2 ? sigmoidf(a.g2[src * a.g2_stride]) : 1.f) : 0.f;
  float ss = 0.f;
  float4 ur[NG];
  if (VEC >= 4) {
#pragma unroll
    for (int it = 0; it < NG; ++it) {
      const int i = 4 * (threadIdx.x + it * blockDim.x);
      if (i >= W) break;
      float4 xv[kMaxStreams];
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < S) xv[s] = ld4<float>(x + s * W + i);
      if (close) {
        float4 yv = float4{0.f, 0.f, 0.f, 0.f};
        if (a.inv) {
          for (int j = 0; j < a.top; ++j) {
            const int row = a.inv[src * a.top + j];
            if (row >= 0) yv = fma4(a.wts[src * a.top + j], ld4<Y>(y + static_cast<int64_t>(row) * W + i), yv);
          }
        } else if (y) {
          yv = ld4<Y>(y + src * W + i);
          for (int sl = 1; sl < a.nslab; ++sl) yv = fma4(1.f, ld4<Y>(y + sl * a.slab_stride + src * W + i), yv);
        }
        if (y2) yv = fma4(gate, ld4<T>(y2 + src * W + i), yv);
        float4 nv[kMaxStreams];
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t) {
          if (t < S) {
            float4 acc = float4{0.f, 0.f, 0.f, 0.f};
            for (int s = 0; s < S; ++s) acc = fma4(c_mix[s * S + t], xv[s], acc);
            nv[t] = fma4(c_out[t], yv, acc);
            st4<float>(x + t * W + i, nv[t]);
          }
        }
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t)
          if (t < S) xv[t] = nv[t];
      }
      if (open) {
        float4 u = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t)
          if (t < S) u = fma4(c_in[t], xv[t], u);
        ur[it] = u;
        ss += (u.x * u.x + u.y * u.y) + (u.z * u.z + u.w * u.w);
      }
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float xv[kMaxStreams];
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) xv[s] = s < S ? x[s * W + i] : 0.f;
      if (close) {
        float yv = 0.f;
        if (a.inv) {
          for (int j = 0; j < a.top; ++j) {
            const int row = a.inv[src * a.top + j];
            if (row >= 0) yv += a.wts[src * a.top + j] * ld<Y>(y + static_cast<int64_t>(row) * W + i);
          }
        } else if (y) {
          yv = ld<Y>(y + src * W + i);
          for (int sl = 1; sl < a.nslab; ++sl) yv += ld<Y>(y + sl * a.slab_stride + src * W + i);
        }
        if (y2) yv += gate * ld<T>(y2 + src * W + i);
        float nv[kMaxStreams];
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t) {
          if (t < S) {
            float acc = 0.f;
            for (int s = 0; s < S; ++s) acc += c_mix[s * S + t] * xv[s];
            nv[t] = acc + c_out[t] * yv;
            x[t * W + i] = nv[t];
          }
        }
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t) xv[t] = t < S ? nv[t] : 0.f;
      }
      if (open) {
        float u = 0.f;
#pragma unroll
        for (int t = 0; t < kMaxStreams; ++t)
          if (t < S) u += c_in[t] * xv[t];
        vbuf[i] = u;
        ss += u * u;
      }
    }
  }
  if (!open) return;
  ss = pk::block_sum(ss, red);
  const float k = 1.f / sqrtf(ss / static_cast<float>(W) + a.eps);
  T* act = static_cast<T*>(a.act);
  if (VEC >= 4) {
#pragma unroll
    for (int it = 0; it < NG; ++it) {
      const int i = 4 * (threadIdx.x + it * blockDim.x);
      if (i >= W) break;
      const float4 u = ur[it], g = ld4<float>(a.norm_w + i);
      const float4 z = float4{u.x * k * g.x, u.y * k * g.y, u.z * k * g.z, u.w * k * g.w};
      if (act) st4<T>(act + static_cast<int64_t>(r) * W + i, z);
      if (a.z32) st4<float>(a.z32 + static_cast<int64_t>(r) * W + i, z);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float z = vbuf[i] * k * a.norm_w[i];
      if (act) st<T>(act + static_cast<int64_t>(r) * W + i, z);
      if (a.z32) a.z32[static_cast<int64_t>(r) * W + i] = z;
    }
  }
}

__global__ void __launch_bounds__(256) tanh_cap_kernel(float* __restrict__ x, int64_t n, float cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

PK_EXPORT int pkm_spread_rows(void* xs, const void* table, const void* ids, int T, int S, int W, int vocab, int dt,
                              float scale, hipStream_t stream) {
  if (T <= 0) return 0;
  if (S < 1 || S > kMaxStreams) return -1;
  PKM_DISPATCH(dt, E, spread_rows_kernel<E><<<T, 256, 0, stream>>>(static_cast<float*>(xs), static_cast<const E*>(table),
                                                                    static_cast<const int*>(ids), S, W, vocab, scale));
  return PK_CHECK_LAUNCH();
}

// xs [tokens, S, W] fp32, updated in place when mix / a_out are given (then y, or inv / wts / y rows,
// is the sublayer output; y_dt its element type, -1: none).  y2 / g2: a second row per token in the
// activation type and its pre-sigmoid gate (fp32, element stride g2_stride; null: the row is added as it is).  a_in / norm_w: open.
// rows: R token indices to open (no close).  act (element type act_dt) and z32 may each be null.
PK_EXPORT int pkm_hyper_step(void* xs, int R, int S, int W, const void* y, int y_dt, int nslab, const void* inv, int top,
                             const void* wts, const void* y2, int y2_dt, const void* g2, long long g2_stride,
                             const void* mix, const void* a_out, const void* a_in, const void* norm_w, float eps,
                             void* act, int act_dt, void* z32, const void* rows, hipStream_t stream) {
  if (R <= 0) return 0;
  if (S < 1 || S > kMaxStreams || W > 16384 || nslab < 1) return -1;
  if ((mix == nullptr) != (a_out == nullptr) || (a_in == nullptr) != (norm_w == nullptr)) return -1;
  if (rows && mix) return -1;
  if (inv && (!y || !wts || top < 1 || nslab > 1)) return -1;
  if (y2 && y2_dt != act_dt) return -1;
  HyperArgs a{static_cast<float*>(xs), S, W, y, nslab, static_cast<int64_t>(R) * W, static_cast<const int*>(inv), top,
              static_cast<const float*>(wts), y2, static_cast<const float*>(g2), g2_stride,
              static_cast<const float*>(mix), static_cast<const float*>(a_out), static_cast<const float*>(a_in),
              static_cast<const float*>(norm_w), eps, act, static_cast<float*>(z32), static_cast<const int*>(rows)};
  const size_t lds = a_in ? static_cast<size_t>(W) * sizeof(float) : 0;
  if (y_dt != kF32 && y_dt != kBF16 && y != nullptr) return -2;
  const bool y32 = y == nullptr || y_dt == kF32;
  if (W % 4 == 0) {  // up to 256 threads, each with 1, 2, 4 or 8 groups of four coordinates
    // prompt-sized launches: eight groups per thread (one wave per token up to 2048 coordinates: no
    // barrier partner to wait for, many tokens and many loads in flight per CU); decode-sized ones:
    // one group per thread, the shortest chain for the few workgroups there are
    const int groups = W / 4;
    const int want = R > 1024 ? (groups + 7) / 8 : groups;
    int threads = (want + 63) / 64 * 64;
    threads = threads > 1024 ? 1024 : threads;
    const int per = (groups + threads - 1) / threads;
#define PKM_HS(YT, VEC) PKM_DISPATCH(act_dt, E, hyper_step_kernel<E, YT, VEC><<<R, threads, 0, stream>>>(a))
#define PKM_HS_Y(VEC)   \
  if (y32) {            \
    PKM_HS(float, VEC); \
  } else {              \
    PKM_HS(bf16_t, VEC); \
  }
    if (per <= 1) {
      PKM_HS_Y(4)
    } else if (per <= 2) {
      PKM_HS_Y(8)
    } else if (per <= 4) {
      PKM_HS_Y(16)
    } else if (per <= 8) {
      PKM_HS_Y(32)
    } else {
      PKM_HS_Y(64)
    }
#undef PKM_HS_Y
#undef PKM_HS
  } else {
    const int threads = W >= 4096 ? 1024 : (W >= 1024 ? 512 : 256);
    if (y32) {
      PKM_DISPATCH(act_dt, E, hyper_step_kernel<E, float, 1><<<R, threads, lds, stream>>>(a));
    } else {
      PKM_DISPATCH(act_dt, E, hyper_step_kernel<E, bf16_t, 1><<<R, threads, lds, stream>>>(a));
    }
  }
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_tanh_cap(void* x, long long n, float cap, hipStream_t stream) {
  if (n <= 0) return 0;
  tanh_cap_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(static_cast<float*>(x), n, cap);
  return PK_CHECK_LAUNCH();
}
