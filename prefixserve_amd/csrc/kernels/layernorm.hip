// Layer norm with weight and bias around the residual stream, and the sinusoid added per position.
//
// LN(y) = (y - mean(y)) / sqrt(mean((y - mean)^2) + eps) * w + b, the mean taken first and the squared
// deviations from it second, all in float. One kernel does what an arrangement with a norm in front of
// and behind every sub-layer needs between two sub-layers:
//     stream[r] += LN_post(delta[r])          (delta: one tensor, or float slices that are summed first)
//     out[r]     = LN_pre(stream[r])          (in the activation type)
// either half may be left out. With a list of rows only the second half runs, on the listed rows.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

// Four neighbouring values at once: a thread asks for all the memory it needs in a few wide loads that
// are in flight together, instead of one value after the other.
template <typename T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4<bf16_t>(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xFFFF0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xFFFF0000u));
}
template <typename T> __device__ __forceinline__ void store4(T* p, float4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float4 v) {
  bf16_t q[4] = {float_to_bf16(v.x), float_to_bf16(v.y), float_to_bf16(v.z), float_to_bf16(v.w)};
  *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(q);
}

// One workgroup of 256 threads per row; the row lies in LDS between its passes. V = 4: the width is a
// multiple of four and every thread handles four neighbouring values at a time; V = 1: any width.
template <typename DT, typename OT, int V>
__global__ __launch_bounds__(256) void layernorm_step_kernel(
    float* __restrict__ residual, const int32_t* __restrict__ rows, const DT* __restrict__ delta, int n_partials,
    int64_t partial_stride, const float* __restrict__ post_w, const float* __restrict__ post_b, float post_eps,
    const float* __restrict__ pre_w, const float* __restrict__ pre_b, float pre_eps, OT* __restrict__ out, int hidden) {
  extern __shared__ __align__(16) float ln_smem[];      // the row, then 4 floats for the sums
  float* row = ln_smem;
  float* scratch = ln_smem + hidden;
  const int64_t r = blockIdx.x;
  const int64_t src = rows != nullptr ? rows[r] : r;
  float* x = residual + src * hidden;
  const float inv_n = 1.f / static_cast<float>(hidden);
  constexpr int kStep = 256 * V;
  if (delta != nullptr) {
    float sum = 0.f;
    const DT* d0 = delta + r * hidden;
#pragma unroll 2
    for (int i = threadIdx.x * V; i < hidden; i += kStep) {
      if constexpr (V == 4) {
        float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
        for (int p = 0; p < n_partials; ++p) {
          const float4 d = load4<DT>(d0 + p * partial_stride + i);
          y.x += d.x, y.y += d.y, y.z += d.z, y.w += d.w;
        }
        *reinterpret_cast<float4*>(row + i) = y;
        sum += (y.x + y.y) + (y.z + y.w);
      } else {
        float y = 0.f;
        for (int p = 0; p < n_partials; ++p) y += to_float<DT>(d0[p * partial_stride + i]);
        row[i] = y;
        sum += y;
      }
    }
    const float mean = block_sum(sum, scratch, 4) * inv_n;
    float sq = 0.f;
    for (int i = threadIdx.x * V; i < hidden; i += kStep) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float d = row[i + e] - mean;
        sq = fmaf(d, d, sq);
      }
    }
    const float inv = 1.f / sqrtf(block_sum(sq, scratch, 4) * inv_n + post_eps);
#pragma unroll 2
    for (int i = threadIdx.x * V; i < hidden; i += kStep) {
      if constexpr (V == 4) {
        const float4 xv = load4<float>(x + i), w = load4<float>(post_w + i), b = load4<float>(post_b + i);
        const float4 y = *reinterpret_cast<const float4*>(row + i);
        const float4 v = make_float4(xv.x + ((y.x - mean) * inv * w.x + b.x), xv.y + ((y.y - mean) * inv * w.y + b.y),
                                     xv.z + ((y.z - mean) * inv * w.z + b.z), xv.w + ((y.w - mean) * inv * w.w + b.w));
        store4<float>(x + i, v);
        *reinterpret_cast<float4*>(row + i) = v;
      } else {
        const float v = x[i] + ((row[i] - mean) * inv * post_w[i] + post_b[i]);
        x[i] = v;
        row[i] = v;
      }
    }
  } else if (out != nullptr) {
#pragma unroll 2
    for (int i = threadIdx.x * V; i < hidden; i += kStep) {
      if constexpr (V == 4) *reinterpret_cast<float4*>(row + i) = load4<float>(x + i);
      else row[i] = x[i];
    }
  }
  if (out == nullptr) return;
  float sum = 0.f;
  for (int i = threadIdx.x * V; i < hidden; i += kStep) {             // every thread reads what it wrote itself
#pragma unroll
    for (int e = 0; e < V; ++e) sum += row[i + e];
  }
  const float mean = block_sum(sum, scratch, 4) * inv_n;
  float sq = 0.f;
  for (int i = threadIdx.x * V; i < hidden; i += kStep) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float d = row[i + e] - mean;
      sq = fmaf(d, d, sq);
    }
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch, 4) * inv_n + pre_eps);
  OT* o = out + r * hidden;
#pragma unroll 2
  for (int i = threadIdx.x * V; i < hidden; i += kStep) {
    if constexpr (V == 4) {
      const float4 w = load4<float>(pre_w + i), b = load4<float>(pre_b + i);
      const float4 y = *reinterpret_cast<const float4*>(row + i);
      store4<OT>(o + i, make_float4((y.x - mean) * inv * w.x + b.x, (y.y - mean) * inv * w.y + b.y,
                                    (y.z - mean) * inv * w.z + b.z, (y.w - mean) * inv * w.w + b.w));
    } else {
      o[i] = from_float<OT>((row[i] - mean) * inv * pre_w[i] + pre_b[i]);
    }
  }
}

// x[t, e] += sin (e even) or cos (e odd) of positions[t] * freq[e / 2]. The angle is formed in double and
// brought into [-pi, pi] there, so that a position in the tens of thousands loses nothing.
__global__ void add_sinusoid_kernel(float* __restrict__ x, const int32_t* __restrict__ positions,
                                    const double* __restrict__ freq, int64_t n, int hidden) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / hidden;
    const int e = static_cast<int>(i - t * hidden);
    double a = static_cast<double>(positions[t]) * freq[e >> 1];
    a -= 6.283185307179586476925 * rint(a * 0.15915494309189533577);
    const float af = static_cast<float>(a);
    x[i] += (e & 1) ? cosf(af) : sinf(af);
  }
}

template <typename DT, typename OT>
static int launch_layernorm(hipStream_t s, float* residual, const int32_t* rows, const void* delta, int n_partials,
                            int64_t partial_stride, const float* post_w, const float* post_b, float post_eps,
                            const float* pre_w, const float* pre_b, float pre_eps, void* out, int64_t n_rows, int hidden) {
  const size_t smem = sizeof(float) * (static_cast<size_t>(hidden) + 4);
  // Four values at a time where every row, slice and parameter starts on a multiple of four values.
  const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool wide = hidden % 4 == 0 && partial_stride % 4 == 0 && aligned(residual) && aligned(delta) && aligned(post_w) &&
                    aligned(post_b) && aligned(pre_w) && aligned(pre_b) && aligned(out);
  const dim3 grid(static_cast<unsigned>(n_rows));
  if (wide) {
    layernorm_step_kernel<DT, OT, 4><<<grid, dim3(256), smem, s>>>(residual, rows, static_cast<const DT*>(delta), n_partials,
                                                                  partial_stride, post_w, post_b, post_eps, pre_w, pre_b,
                                                                  pre_eps, static_cast<OT*>(out), hidden);
  } else {
    layernorm_step_kernel<DT, OT, 1><<<grid, dim3(256), smem, s>>>(residual, rows, static_cast<const DT*>(delta), n_partials,
                                                                  partial_stride, post_w, post_b, post_eps, pre_w, pre_b,
                                                                  pre_eps, static_cast<OT*>(out), hidden);
  }
  return check_launch("psamd_layernorm_step");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_layernorm_step(void* stream, float* residual, const int32_t* rows, const void* delta, int delta_dtype,
                         int n_partials, int64_t partial_stride, const float* post_w, const float* post_b, float post_eps,
                         const float* pre_w, const float* pre_b, float pre_eps, void* out, int out_dtype, int64_t n_rows,
                         int hidden) {
  PSAMD_REQUIRE(n_rows >= 0 && hidden > 0 && n_rows <= 2147483647LL, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * (static_cast<size_t>(hidden) + 4) <= 64 * 1024, "a row does not fit in LDS");
  PSAMD_REQUIRE(delta == nullptr || (post_w != nullptr && post_b != nullptr && n_partials >= 1 && rows == nullptr),
                "a delta needs the norm behind it, and all rows");
  PSAMD_REQUIRE(out == nullptr || (pre_w != nullptr && pre_b != nullptr), "an output needs the norm in front of it");
  PSAMD_REQUIRE(delta != nullptr || out != nullptr, "nothing to do");
  PSAMD_REQUIRE(n_partials <= 1 || delta_dtype == kF32, "partial sums are float32");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool dbf = delta != nullptr && delta_dtype == kBF16;
  const bool obf = out != nullptr && out_dtype == kBF16;
  if (delta != nullptr && delta_dtype != kBF16 && delta_dtype != kF32) return fail("psamd_layernorm_step: bad delta dtype");
  if (out != nullptr && out_dtype != kBF16 && out_dtype != kF32) return fail("psamd_layernorm_step: bad output dtype");
  if (dbf && obf)
    return launch_layernorm<bf16_t, bf16_t>(s, residual, rows, delta, n_partials, partial_stride, post_w, post_b, post_eps,
                                            pre_w, pre_b, pre_eps, out, n_rows, hidden);
  if (dbf)
    return launch_layernorm<bf16_t, float>(s, residual, rows, delta, n_partials, partial_stride, post_w, post_b, post_eps,
                                           pre_w, pre_b, pre_eps, out, n_rows, hidden);
  if (obf)
    return launch_layernorm<float, bf16_t>(s, residual, rows, delta, n_partials, partial_stride, post_w, post_b, post_eps,
                                           pre_w, pre_b, pre_eps, out, n_rows, hidden);
  return launch_layernorm<float, float>(s, residual, rows, delta, n_partials, partial_stride, post_w, post_b, post_eps, pre_w,
                                        pre_b, pre_eps, out, n_rows, hidden);
}

int psamd_add_sinusoid(void* stream, float* x, const int32_t* positions, const double* freq, int64_t tokens, int hidden) {
  PSAMD_REQUIRE(tokens >= 0 && hidden > 0, "bad sizes");
  if (tokens == 0) return 0;
  const int64_t n = tokens * hidden;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(n, 256), 65535));
  add_sinusoid_kernel<<<dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, positions, freq, n, hidden);
  return check_launch("psamd_add_sinusoid");
}

}  // extern "C"
