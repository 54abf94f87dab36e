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

// One workgroup of 256 threads per row; the row lies in LDS between its passes.
template <typename DT, typename OT>
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
  if (delta != nullptr) {
    float sum = 0.f;
    for (int i = threadIdx.x; i < hidden; i += 256) {
      float y = 0.f;
      for (int p = 0; p < n_partials; ++p) y += to_float<DT>(delta[p * partial_stride + r * hidden + i]);
      row[i] = y;
      sum += y;
    }
    const float mean = block_sum(sum, scratch, 4) * inv_n;
    float sq = 0.f;
    for (int i = threadIdx.x; i < hidden; i += 256) {
      const float d = row[i] - mean;
      sq = fmaf(d, d, sq);
    }
    const float inv = 1.f / sqrtf(block_sum(sq, scratch, 4) * inv_n + post_eps);
    for (int i = threadIdx.x; i < hidden; i += 256) {
      const float v = x[i] + ((row[i] - mean) * inv * post_w[i] + post_b[i]);
      x[i] = v;
      row[i] = v;
    }
  } else if (out != nullptr) {
    for (int i = threadIdx.x; i < hidden; i += 256) row[i] = x[i];
  }
  if (out == nullptr) return;
  float sum = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) sum += row[i];      // every thread reads what it wrote itself
  const float mean = block_sum(sum, scratch, 4) * inv_n;
  float sq = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float d = row[i] - mean;
    sq = fmaf(d, d, sq);
  }
  const float inv = 1.f / sqrtf(block_sum(sq, scratch, 4) * inv_n + pre_eps);
  OT* o = out + r * hidden;
  for (int i = threadIdx.x; i < hidden; i += 256) o[i] = from_float<OT>((row[i] - mean) * inv * pre_w[i] + pre_b[i]);
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
  layernorm_step_kernel<DT, OT><<<dim3(static_cast<unsigned>(n_rows)), dim3(256), smem, s>>>(
      residual, rows, static_cast<const DT*>(delta), n_partials, partial_stride, post_w, post_b, post_eps, pre_w, pre_b,
      pre_eps, static_cast<OT*>(out), hidden);
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
