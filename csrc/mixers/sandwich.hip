// An fp32 residual stream whose sublayers sit between two layer norms (weight and bias each).
//
//   sandwich_step   closes one sublayer and opens the next, per token, in one pass:
//                     z = the sublayer's output row (a plain row or the sum of split-K slabs)
//                     z <- LN(z) * pw + pb                       when a norm follows the sublayer
//                     x <- x + z        or  x <- z + add         (`replace`: a block's re-projection)
//                     act = LN(x) * ow + ob                      the next sublayer's input
//                   either half may be absent; with `rows` only those tokens are opened.
//                   LN(v) = (v - mean) / sqrt(mean((v - mean)^2) + eps), two passes over the row in fp32.
//   join_cast       out[t] = [x[t] | x0[t]] in the activation type
//   silu_mul        out = silu(gate) * up of [gate | up] rows (or their split-K slabs), product in fp32
//   scale           x <- k x
//
// One workgroup per token; every sum runs in a fixed order, so a token's result does not depend
// on the rest of the batch.
#include "mix_common.h"

using namespace pkm;

namespace {

constexpr int kThreads = 256;
constexpr int kMaxPer = 16;  // row values per thread: rows of up to 4096 numbers stay in registers

struct SandwichArgs {
  float* x;
  int W;
  const void* y;
  int nslab;
  int64_t slab_stride;
  const float* pw;
  const float* pb;
  int replace;
  const float* add;
  const float* ow;
  const float* ob;
  float eps;
  void* act;
  const int* rows;
};

// mean and 1 / sqrt(var + eps) of the row held as v[i] = row[tid + i * kThreads] (REG) or in `buf`
template <bool REG>
__device__ __forceinline__ void row_stats(const float* v, const float* buf, int W, float eps, float* red, float& mean,
                                          float& rstd) {
  float s = 0.f;
  if (REG) {
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) s += v[i];
  } else {
    for (int i = threadIdx.x; i < W; i += kThreads) s += buf[i];
  }
  mean = pk::block_sum(s, red) / static_cast<float>(W);
  float q = 0.f;
  if (REG) {
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
      const float d = (static_cast<int>(threadIdx.x) + i * kThreads < W) ? v[i] - mean : 0.f;
      q += d * d;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += kThreads) {
      const float d = buf[i] - mean;
      q += d * d;
    }
  }
  rstd = 1.f / sqrtf(pk::block_sum(q, red) / static_cast<float>(W) + eps);
}

// YT: element type of y (float for slabs), AT: element type of act.  REG: W <= kMaxPer * kThreads.
template <typename YT, typename AT, bool REG>
__global__ void __launch_bounds__(kThreads) sandwich_kernel(SandwichArgs a) {
  extern __shared__ float buf[];  // [W] when !REG
  __shared__ float red[16];
  const int r = blockIdx.x, tid = threadIdx.x, W = a.W;
  const int t = a.rows ? a.rows[r] : r;
  float* xr = a.x + static_cast<int64_t>(t) * W;
  float v[kMaxPer];
  float mean, rstd;
  if (a.y) {
    const YT* yr = static_cast<const YT*>(a.y) + static_cast<int64_t>(t) * W;
    auto get = [&](int c) {
      float z = ld<YT>(yr + c);
      for (int s = 1; s < a.nslab; ++s) z += ld<YT>(yr + s * a.slab_stride + c);
      return z;
    };
    if (REG) {
#pragma unroll
      for (int i = 0; i < kMaxPer; ++i) {
        const int c = tid + i * kThreads;
        v[i] = c < W ? get(c) : 0.f;
      }
    } else {
      for (int c = tid; c < W; c += kThreads) buf[c] = get(c);
      __syncthreads();
    }
    if (a.pw) {
      row_stats<REG>(v, buf, W, a.eps, red, mean, rstd);
    } else {
      mean = 0.f;
      rstd = 1.f;
    }
    auto fold = [&](int c, float z) {
      if (a.pw) z = (z - mean) * rstd * a.pw[c] + a.pb[c];
      z = a.replace ? z + (a.add ? a.add[c] : 0.f) : xr[c] + z;
      xr[c] = z;
      return z;
    };
    if (REG) {
#pragma unroll
      for (int i = 0; i < kMaxPer; ++i) {
        const int c = tid + i * kThreads;
        v[i] = c < W ? fold(c, v[i]) : 0.f;
      }
    } else {
      for (int c = tid; c < W; c += kThreads) buf[c] = fold(c, buf[c]);
      __syncthreads();
    }
  } else if (a.ow) {
    if (REG) {
#pragma unroll
      for (int i = 0; i < kMaxPer; ++i) {
        const int c = tid + i * kThreads;
        v[i] = c < W ? xr[c] : 0.f;
      }
    } else {
      for (int c = tid; c < W; c += kThreads) buf[c] = xr[c];
      __syncthreads();
    }
  }
  if (!a.ow) return;
  row_stats<REG>(v, buf, W, a.eps, red, mean, rstd);
  AT* out = static_cast<AT*>(a.act) + static_cast<int64_t>(r) * W;
  if (REG) {
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
      const int c = tid + i * kThreads;
      if (c < W) st<AT>(out + c, (v[i] - mean) * rstd * a.ow[c] + a.ob[c]);
    }
  } else {
    for (int c = tid; c < W; c += kThreads) st<AT>(out + c, (buf[c] - mean) * rstd * a.ow[c] + a.ob[c]);
  }
}

template <typename E>
__device__ __forceinline__ float4 ld4(const E* p);
template <>
__device__ __forceinline__ float4 ld4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <>
__device__ __forceinline__ float4 ld4<bf16_t>(const bf16_t* p) {
  const uint2 w = *reinterpret_cast<const uint2*>(p);
  return float4{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                __uint_as_float(w.y & 0xffff0000u)};
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

// The same step for W % 4 == 0, W <= 4 * kVecGroups * kThreads: four consecutive coordinates per
// thread and group, 16-byte accesses of the fp32 rows, the row stays in registers between passes.
constexpr int kVecGroups = 4;

template <typename YT, typename AT>
__global__ void __launch_bounds__(kThreads) sandwich_vec_kernel(SandwichArgs a) {
  __shared__ float red[16];
  const int r = blockIdx.x, tid = threadIdx.x, W = a.W;
  const int t = a.rows ? a.rows[r] : r;
  float* xr = a.x + static_cast<int64_t>(t) * W;
  float4 v[kVecGroups];
  auto stats = [&](float& mean, float& rstd) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < kVecGroups; ++g) s += (v[g].x + v[g].y) + (v[g].z + v[g].w);
    mean = pk::block_sum(s, red) / static_cast<float>(W);
    float q = 0.f;
#pragma unroll
    for (int g = 0; g < kVecGroups; ++g) {
      if (4 * (tid + g * kThreads) < W) {
        const float d0 = v[g].x - mean, d1 = v[g].y - mean, d2 = v[g].z - mean, d3 = v[g].w - mean;
        q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      }
    }
    rstd = 1.f / sqrtf(pk::block_sum(q, red) / static_cast<float>(W) + a.eps);
  };
  auto norm4 = [](float4 z, float mean, float rstd, float4 w, float4 b) {
    return float4{(z.x - mean) * rstd * w.x + b.x, (z.y - mean) * rstd * w.y + b.y, (z.z - mean) * rstd * w.z + b.z,
                  (z.w - mean) * rstd * w.w + b.w};
  };
  float mean = 0.f, rstd = 1.f;
  if (a.y) {
    const YT* yr = static_cast<const YT*>(a.y) + static_cast<int64_t>(t) * W;
#pragma unroll
    for (int g = 0; g < kVecGroups; ++g) {
      const int c = 4 * (tid + g * kThreads);
      v[g] = float4{0.f, 0.f, 0.f, 0.f};
      if (c < W) {
        v[g] = ld4<YT>(yr + c);
        for (int s = 1; s < a.nslab; ++s) {
          const float4 z = ld4<YT>(yr + s * a.slab_stride + c);
          v[g].x += z.x, v[g].y += z.y, v[g].z += z.z, v[g].w += z.w;
        }
      }
    }
    if (a.pw) stats(mean, rstd);
#pragma unroll
    for (int g = 0; g < kVecGroups; ++g) {
      const int c = 4 * (tid + g * kThreads);
      if (c < W) {
        float4 z = v[g];
        if (a.pw) z = norm4(z, mean, rstd, ld4<float>(a.pw + c), ld4<float>(a.pb + c));
        if (a.replace) {
          if (a.add) {
            const float4 d = ld4<float>(a.add + c);
            z.x += d.x, z.y += d.y, z.z += d.z, z.w += d.w;
          }
        } else {
          const float4 x = ld4<float>(xr + c);
          z.x += x.x, z.y += x.y, z.z += x.z, z.w += x.w;
        }
        st4<float>(xr + c, z);
        v[g] = z;
      }
    }
  } else {
#pragma unroll
    for (int g = 0; g < kVecGroups; ++g) {
      const int c = 4 * (tid + g * kThreads);
      v[g] = c < W ? ld4<float>(xr + c) : float4{0.f, 0.f, 0.f, 0.f};
    }
  }
  if (!a.ow) return;
  stats(mean, rstd);
  AT* out = static_cast<AT*>(a.act) + static_cast<int64_t>(r) * W;
#pragma unroll
  for (int g = 0; g < kVecGroups; ++g) {
    const int c = 4 * (tid + g * kThreads);
    if (c < W) st4<AT>(out + c, norm4(v[g], mean, rstd, ld4<float>(a.ow + c), ld4<float>(a.ob + c)));
  }
}

template <typename YT, typename AT>
int launch_sandwich(const SandwichArgs& a, int R, hipStream_t stream) {
  if (a.W % 4 == 0 && a.W <= 4 * kVecGroups * kThreads) {
    sandwich_vec_kernel<YT, AT><<<R, kThreads, 0, stream>>>(a);
  } else if (a.W <= kMaxPer * kThreads) {
    sandwich_kernel<YT, AT, true><<<R, kThreads, 0, stream>>>(a);
  } else {
    sandwich_kernel<YT, AT, false><<<R, kThreads, static_cast<size_t>(a.W) * sizeof(float), stream>>>(a);
  }
  return PK_CHECK_LAUNCH();
}

template <typename T>
__global__ void __launch_bounds__(256) join_cast_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                        const float* __restrict__ x0, int W) {
  const int64_t t = blockIdx.x;
  T* dst = out + t * 2 * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    st<T>(dst + c, x[t * W + c]);
    st<T>(dst + W + c, x0[t * W + c]);
  }
}

template <typename IN, typename T>
__global__ void __launch_bounds__(256) silu_mul_kernel(T* __restrict__ out, const IN* __restrict__ gu, int F, int nslab,
                                                       int64_t slab_stride) {
  const int64_t t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= F) return;
  const IN* row = gu + t * 2 * F;
  float g = ld<IN>(row + c), u = ld<IN>(row + F + c);
  for (int s = 1; s < nslab; ++s) {
    g += ld<IN>(row + s * slab_stride + c);
    u += ld<IN>(row + s * slab_stride + F + c);
  }
  st<T>(out + t * F + c, g / (1.f + expf(-g)) * u);
}

template <typename IN, typename T>
__global__ void __launch_bounds__(256) silu_mul_vec_kernel(T* __restrict__ out, const IN* __restrict__ gu, int F, int nslab,
                                                           int64_t slab_stride) {
  const int64_t t = blockIdx.y;
  const int c = 4 * (blockIdx.x * blockDim.x + threadIdx.x);
  if (c >= F) return;
  const IN* row = gu + t * 2 * F;
  float4 g = ld4<IN>(row + c), u = ld4<IN>(row + F + c);
  for (int s = 1; s < nslab; ++s) {
    const float4 g2 = ld4<IN>(row + s * slab_stride + c), u2 = ld4<IN>(row + s * slab_stride + F + c);
    g.x += g2.x, g.y += g2.y, g.z += g2.z, g.w += g2.w;
    u.x += u2.x, u.y += u2.y, u.z += u2.z, u.w += u2.w;
  }
  auto f = [](float gg, float uu) { return gg / (1.f + expf(-gg)) * uu; };
  st4<T>(out + t * F + c, float4{f(g.x, u.x), f(g.y, u.y), f(g.z, u.z), f(g.w, u.w)});
}

__global__ void __launch_bounds__(256) scale_kernel(float* __restrict__ x, int64_t n, float k) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) x[i] *= k;
}

}  // namespace

// x [tokens, W] fp32, updated in place when y is given (y_dt its element type, -1: none; nslab > 1:
// fp32 slabs [nslab][R][W]).  pw / pb: the norm behind the sublayer (null: y is added as it is).
// replace: x <- y (+ add [W]).  ow / ob: open into act (element type act_dt).  rows: R token indices
// to open (no y).
PK_EXPORT int pkm_sandwich_step(void* x, int R, int W, const void* y, int y_dt, int nslab, const void* pw, const void* pb,
                                int replace, const void* add, const void* ow, const void* ob, float eps, void* act,
                                int act_dt, const void* rows, hipStream_t stream) {
  if (R <= 0) return 0;
  if (W < 1 || W > 15360 || nslab < 1) return -1;
  if ((pw == nullptr) != (pb == nullptr) || (ow == nullptr) != (ob == nullptr) || (ow != nullptr) != (act != nullptr)) return -1;
  if ((rows && y) || (nslab > 1 && y_dt != kF32) || (!y && !ow)) return -1;
  SandwichArgs a{static_cast<float*>(x), W, y, nslab, static_cast<int64_t>(R) * W, static_cast<const float*>(pw),
                 static_cast<const float*>(pb), replace, static_cast<const float*>(add), static_cast<const float*>(ow),
                 static_cast<const float*>(ob), eps, act, static_cast<const int*>(rows)};
  if (!y || y_dt == kF32) {
    PKM_DISPATCH(act_dt, A, return (launch_sandwich<float, A>(a, R, stream)));
  }
  if (y_dt != kBF16) return -2;
  PKM_DISPATCH(act_dt, A, return (launch_sandwich<bf16_t, A>(a, R, stream)));
  return 0;
}

PK_EXPORT int pkm_join_cast(void* out, const void* x, const void* x0, int T, int W, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  PKM_DISPATCH(dt, E, join_cast_kernel<E><<<T, 256, 0, stream>>>(static_cast<E*>(out), static_cast<const float*>(x),
                                                                  static_cast<const float*>(x0), W));
  return PK_CHECK_LAUNCH();
}

// gu [T, 2F] (in_dt; nslab > 1: fp32 slabs [nslab][T][2F]) -> out [T, F] (out_dt)
PK_EXPORT int pkm_silu_mul(void* out, const void* gu, int T, int F, int nslab, int in_dt, int out_dt, hipStream_t stream) {
  if (T <= 0 || F <= 0) return 0;
  if (nslab < 1 || (nslab > 1 && in_dt != kF32)) return -1;
  const int64_t ss = static_cast<int64_t>(T) * 2 * F;
  if (F % 4 == 0) {
    const dim3 vgrid((F / 4 + 255) / 256, T);
    if (in_dt == kF32) {
      PKM_DISPATCH(out_dt, E, silu_mul_vec_kernel<float, E><<<vgrid, 256, 0, stream>>>(
                                  static_cast<E*>(out), static_cast<const float*>(gu), F, nslab, ss));
    } else if (in_dt == kBF16) {
      PKM_DISPATCH(out_dt, E, silu_mul_vec_kernel<bf16_t, E><<<vgrid, 256, 0, stream>>>(
                                  static_cast<E*>(out), static_cast<const bf16_t*>(gu), F, 1, ss));
    } else {
      return -2;
    }
    return PK_CHECK_LAUNCH();
  }
  const dim3 grid((F + 255) / 256, T);
  if (in_dt == kF32) {
    PKM_DISPATCH(out_dt, E, silu_mul_kernel<float, E><<<grid, 256, 0, stream>>>(static_cast<E*>(out),
                                                                                 static_cast<const float*>(gu), F, nslab, ss));
  } else if (in_dt == kBF16) {
    PKM_DISPATCH(out_dt, E, silu_mul_kernel<bf16_t, E><<<grid, 256, 0, stream>>>(static_cast<E*>(out),
                                                                                  static_cast<const bf16_t*>(gu), F, 1, ss));
  } else {
    return -2;
  }
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_scale(void* x, long long n, float k, hipStream_t stream) {
  if (n <= 0) return 0;
  scale_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(static_cast<float*>(x), n, k);
  return PK_CHECK_LAUNCH();
}
