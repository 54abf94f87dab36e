// Several copies of the residual stream, mixers side by side, a feed-forward without a gate, and the
// operands of two recurrences that run through the delta rules' scan:
//   * stream_rms_norm: an RMS norm on float rows in place;
//   * hyper_read / hyper_write: a sub-layer reads a weighted sum of the copies through an RMS norm and
//     writes every copy from a mix of the old ones plus its own output;
//   * weighted_sum: a * x + b * y of two sub-layer outputs (each one tensor or float slices);
//   * activation: an elementwise function in place;
//   * gated_group_norm: (y + skip x) silu(z), an RMS norm in equal parts, a weight;
//   * state_space_prepare: step size and decay of a selective state space layer;
//   * matrix_memory_gates / _operands / memory_read_norm_gate: a matrix memory's exponential gates with
//     their running maximum, its operands as float vectors, and its read-out behind the scan;
//   * pool_kv_append: the mean key and value of a block of tokens, written to a page of its own.
// Everything here is float arithmetic; rows in the activation type are widened when read.

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kMaxStreams = 16;

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// grid (rows), 256 threads.
__global__ __launch_bounds__(256) void stream_rms_norm_kernel(float* __restrict__ x, const float* __restrict__ w, float eps,
                                                              int hidden) {
  __shared__ float scratch[4];
  float* row = x + static_cast<int64_t>(blockIdx.x) * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) ss = fmaf(row[i], row[i], ss);
  ss = block_sum(ss, scratch, 4);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += 256) row[i] = row[i] * inv * w[i];
}

// grid (tokens), 256 threads: u = sum_s read[s] streams[s, t, :]; out = u / rms(u) * w (* factor). u is formed
// once and kept in LDS (hidden floats) between the sum of squares and the output. COUNT > 0: the number of streams
// is known at compile time, so that a thread's loads of all streams are in flight together (a step of a few
// tokens is a few workgroups, and what it costs is how many loads wait for one another); COUNT 0: any number.
template <typename O, int COUNT>
__global__ __launch_bounds__(256) void hyper_read_kernel(const float* __restrict__ streams, int64_t stream_stride, int count,
                                                         const float* __restrict__ read, const float* __restrict__ w, float eps,
                                                         const float* __restrict__ factor, O* __restrict__ out, int hidden) {
  __shared__ float scratch[4];
  extern __shared__ float u_s[];
  const float* base = streams + static_cast<int64_t>(blockIdx.x) * hidden;
  constexpr int N = COUNT > 0 ? COUNT : kMaxStreams;
  const int n = COUNT > 0 ? COUNT : count;
  float a[N];
#pragma unroll
  for (int s = 0; s < N; ++s) a[s] = s < n ? read[s] : 0.f;
  float ss = 0.f;
  for (int i0 = threadIdx.x; i0 < hidden; i0 += 1024) {
    float u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + 256 * j;
      if (i < hidden) {
#pragma unroll
        for (int s = 0; s < N; ++s)
          if (s < n) u[j] = fmaf(a[s], base[s * stream_stride + i], u[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + 256 * j;
      if (i < hidden) {
        u_s[i] = u[j];
        ss = fmaf(u[j], u[j], ss);
      }
    }
  }
  ss = block_sum(ss, scratch, 4);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(hidden) + eps);
  O* o = out + static_cast<int64_t>(blockIdx.x) * hidden;
  for (int i = threadIdx.x; i < hidden; i += 256) {       // a thread reads back what it wrote itself
    float v = u_s[i] * inv * w[i];
    if (factor != nullptr) v *= factor[i];
    o[i] = from_float<O>(v);
  }
}

__device__ __forceinline__ float delta_at(const void* d, int dtype, int slices, int64_t stride, int64_t e) {
  if (slices > 1 || dtype == kF32) {
    const float* f = static_cast<const float*>(d);
    float y = f[e];
    for (int s = 1; s < slices; ++s) y += f[s * stride + e];
    return y;
  }
  return bf16_to_float(static_cast<const bf16_t*>(d)[e]);
}

// One thread per (token, channel): new[t] = sum_s mix[s, t] old[s] + write[t] * y, y = a_scale * a (+ b_scale * b): each
// one tensor in its dtype, or float slices a stride apart, added in ascending order.
__global__ __launch_bounds__(256) void hyper_write_kernel(float* __restrict__ streams, int64_t stream_stride, int count,
                                                          const float* __restrict__ mix, const float* __restrict__ write,
                                                          const void* __restrict__ a, int a_dtype, int a_slices, int64_t a_stride,
                                                          float a_scale, const void* __restrict__ b, int b_dtype, int b_slices,
                                                          int64_t b_stride, float b_scale, int64_t n) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= n) return;
  float y = a_scale * delta_at(a, a_dtype, a_slices, a_stride, e);
  if (b != nullptr) y = fmaf(b_scale, delta_at(b, b_dtype, b_slices, b_stride, e), y);
  float old[kMaxStreams];
#pragma unroll
  for (int s = 0; s < kMaxStreams; ++s) old[s] = s < count ? streams[s * stream_stride + e] : 0.f;
#pragma unroll
  for (int t = 0; t < kMaxStreams; ++t) {
    if (t < count) {
      float v = write[t] * y;
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < count) v = fmaf(mix[s * count + t], old[s], v);
      streams[t * stream_stride + e] = v;
    }
  }
}

__global__ __launch_bounds__(256) void weighted_sum_kernel(const void* __restrict__ a, int a_dtype, int a_slices, int64_t a_stride,
                                                           float a_scale, const void* __restrict__ b, int b_dtype, int b_slices,
                                                           int64_t b_stride, float b_scale, float* __restrict__ out, int64_t n) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= n) return;
  out[e] = fmaf(a_scale, delta_at(a, a_dtype, a_slices, a_stride, e), b_scale * delta_at(b, b_dtype, b_slices, b_stride, e));
}

// kind 0 = GELU (exact), 1 = GELU (tanh form), 2 = SiLU, 3 = ReLU.
__device__ __forceinline__ float activate(float z, int kind) {
  if (kind == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
  if (kind == 1) return gelu_tanh_f(z);
  if (kind == 2) return z * sigmoid_f(z);
  return fmaxf(z, 0.f);
}

// Sixteen bytes per thread and access (8 bfloat16 or 4 floats); the entries behind the last whole group one by one.
template <typename A>
__global__ __launch_bounds__(256) void activation_kernel(A* __restrict__ x, int64_t n, int kind) {
  constexpr int V = 16 / sizeof(A);
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t groups = n / V;
  if (g < groups) {
    uint4 raw = reinterpret_cast<uint4*>(x)[g];
    A* v = reinterpret_cast<A*>(&raw);
#pragma unroll
    for (int i = 0; i < V; ++i) v[i] = from_float<A>(activate(to_float<A>(v[i]), kind));
    reinterpret_cast<uint4*>(x)[g] = raw;
  } else if (g == groups) {
    for (int64_t e = groups * V; e < n; ++e) x[e] = from_float<A>(activate(to_float<A>(x[e]), kind));
  }
}

// v = (y + skip[head] x) * silu(z); out = v / sqrt(mean(v^2) + eps) * weight over each of `parts` equal parts of a row.
// WAVES = 1: one wave per (token, part), four of them a workgroup; WAVES = 4: a whole workgroup per (token, part), for
// parts of more than 256 entries (a row normalized as a whole by one wave is 64 rounds of loads in a row).
template <typename A, int WAVES>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ x,
                                                               int64_t x_row, const float* __restrict__ skip, int vdim,
                                                               const A* __restrict__ gate, int64_t gate_row,
                                                               const float* __restrict__ weight, int parts, int part, float eps,
                                                               A* __restrict__ out, int64_t pairs) {
  __shared__ float scratch[4];
  constexpr int T = WAVES * kWave;
  const int lane = threadIdx.x % T;
  const int64_t pair = WAVES == 4 ? static_cast<int64_t>(blockIdx.x) : static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;                       // with WAVES = 4 the whole workgroup leaves together
  const int64_t t = pair / parts;
  const int c0 = static_cast<int>(pair - t * parts) * part;
  const int64_t inner = static_cast<int64_t>(parts) * part;
  float ss = 0.f;
  for (int i = lane; i < part; i += T) {
    const int c = c0 + i;
    const float z = to_float<A>(gate[t * gate_row + c]);
    const float v = fmaf(skip[c / vdim], x[t * x_row + c], y[t * inner + c]) * z * sigmoid_f(z);
    ss = fmaf(v, v, ss);
  }
  ss = WAVES == 4 ? block_sum(ss, scratch, 4) : wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(part) + eps);
  for (int i = lane; i < part; i += T) {
    const int c = c0 + i;
    const float z = to_float<A>(gate[t * gate_row + c]);
    const float v = fmaf(skip[c / vdim], x[t * x_row + c], y[t * inner + c]) * z * sigmoid_f(z);
    out[t * inner + c] = from_float<A>(v * inv * weight[c]);
  }
}

// coef row = [exp(-exp(a_log[h]) d) | 0 | d], d = softplus(dt[t, h] + dt_bias[h]).
__global__ __launch_bounds__(256) void state_space_prepare_kernel(const float* __restrict__ dt, const float* __restrict__ dt_bias,
                                                                  const float* __restrict__ a_log, float* __restrict__ coef,
                                                                  int64_t n, int heads) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= n) return;
  const int64_t t = e / heads;
  const int h = static_cast<int>(e - t * heads);
  const float d = softplus_f(dt[e] + dt_bias[h]);
  float* c = coef + t * 3 * heads;
  c[h] = expf(-expf(a_log[h]) * d);
  c[heads + h] = 0.f;
  c[2 * heads + h] = d;
}

// grid (items, heads), one wave: the gates of a matrix memory with their running maximum m. gates row =
// [input | forget] inputs (heads each); i = cap tanh((. + b) / cap), f = logsigmoid(cap tanh(.));
// m' = max(f + m, i); coef row = [exp(f + m - m') | 0 | exp(i - m') | exp(-m')]; m lives in the item's slot.
// A token is the map m -> max(m + f, i); two of them in a row are the map m -> max(m + (f1 + f2), max(i1 + f2, i2)),
// so 64 tokens at a time are put together by a scan over the wave's lanes and applied to the m in front of them.
__global__ __launch_bounds__(64) void matrix_memory_gates_kernel(const float* __restrict__ gates, const float* __restrict__ bias,
                                                                 float cap, float* __restrict__ coef, float* __restrict__ state,
                                                                 int64_t state_row, const int32_t* __restrict__ item_start,
                                                                 const int32_t* __restrict__ slots, int heads) {
  const int item = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t s0 = item_start[item], s1 = item_start[item + 1];
  float* mp = state + static_cast<int64_t>(slots[item]) * state_row + h;
  float m = *mp;
  const float bi = bias[h], bf = bias[heads + h];
  for (int64_t t0 = s0; t0 < s1; t0 += kWave) {
    const int64_t t = t0 + lane;
    const bool valid = t < s1;
    // A lane past the item's end is the map that changes nothing.
    const float il = valid ? cap * tanhf((gates[t * 2 * heads + h] + bi) / cap) : -INFINITY;
    const float fl = valid ? -softplus_f(-cap * tanhf((gates[t * 2 * heads + heads + h] + bf) / cap)) : 0.f;
    float a = fl, b = il;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const float ap = __shfl_up(a, o, kWave), bp = __shfl_up(b, o, kWave);
      if (lane >= o) {
        b = fmaxf(bp + a, b);
        a = ap + a;
      }
    }
    const float mn = fmaxf(m + a, b);
    float before = __shfl_up(mn, 1, kWave);
    if (lane == 0) before = m;
    if (valid) {
      float* c = coef + t * 4 * heads;
      c[h] = expf(fl + before - mn);
      c[heads + h] = 0.f;
      c[2 * heads + h] = expf(il - mn);
      c[3 * heads + h] = expf(-mn);
    }
    m = __shfl(mn, kWave - 1, kWave);
  }
  if (lane == 0) *mp = m;
}

// grid (tokens), 256 threads: u row = [q * q_scale | k] (heads x dim each), vals row = per head [v | 1].
template <typename A>
__global__ __launch_bounds__(256) void matrix_memory_operands_kernel(const A* __restrict__ rows, int64_t in_row, int q_col, int k_col,
                                                                     int v_col, int heads, int dim, int vdim, float q_scale,
                                                                     float* __restrict__ u, float* __restrict__ vals) {
  const int64_t t = blockIdx.x;
  const A* r = rows + t * in_row;
  const int hd = heads * dim;
  for (int i = threadIdx.x; i < hd; i += 256) {
    u[t * 2 * hd + i] = to_float<A>(r[q_col + i]) * q_scale;
    u[t * 2 * hd + hd + i] = to_float<A>(r[k_col + i]);
  }
  const int hv = heads * (vdim + 1);
  for (int i = threadIdx.x; i < hv; i += 256) {
    const int h = i / (vdim + 1), j = i - h * (vdim + 1);
    vals[t * hv + i] = j < vdim ? to_float<A>(r[v_col + h * vdim + j]) : 1.f;
  }
}

// One wave per (token, head): raw = [S^T q : vdim | n . q]; o = raw / (max(|n . q|, floor) + read_eps);
// out = o / sqrt(mean(o^2) + eps) * weight[h, :] * sigmoid(gate).
template <typename A>
__global__ __launch_bounds__(256) void memory_read_norm_gate_kernel(const float* __restrict__ raw, const float* __restrict__ floor_,
                                                                    int64_t floor_row, int heads, int vdim, float read_eps,
                                                                    const float* __restrict__ weight, float eps,
                                                                    const A* __restrict__ gate, int64_t gate_row,
                                                                    A* __restrict__ out, int64_t pairs) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t pair = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int64_t t = pair / heads;
  const int h = static_cast<int>(pair - t * heads);
  const float* src = raw + pair * (vdim + 1);
  const float den = fmaxf(fabsf(src[vdim]), floor_[t * floor_row + h]) + read_eps;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += kWave) {
    const float o = src[i] / den;
    ss = fmaf(o, o, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(vdim) + eps);
  for (int i = lane; i < vdim; i += kWave) {
    const float z = to_float<A>(gate[t * gate_row + static_cast<int64_t>(h) * vdim + i]);
    out[pair * vdim + i] = from_float<A>(src[i] / den * inv * weight[static_cast<int64_t>(h) * vdim + i] * sigmoid_f(z));
  }
}

// grid (tokens, kv heads), 64 threads. A token whose pool_slot is >= 0 completes a block of `block`
// tokens: the mean of their keys ([16][d] halves of the token pages) and values ([d][16]) goes to
// place pool_slot of the pool's pages, summed in float in the order of the positions.
template <typename A>
__global__ __launch_bounds__(64) void pool_kv_append_kernel(const A* __restrict__ kv, A* __restrict__ pool,
                                                            const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_item,
                                                            const int32_t* __restrict__ table_off, const int32_t* __restrict__ block_ids,
                                                            const int32_t* __restrict__ pool_slot, int hkv, int d, int block) {
  const int64_t t = blockIdx.x;
  const int slot = pool_slot[t];
  if (slot < 0) return;
  const int kvh = blockIdx.y;
  const int pos = positions[t];
  const int32_t* table = block_ids + table_off[tok_item[t]];
  const int64_t page_elems = 2LL * hkv * kPage * d, half = static_cast<int64_t>(hkv) * kPage * d;
  const float inv = 1.f / static_cast<float>(block);
  A* dst = pool + static_cast<int64_t>(slot / kPage) * page_elems + static_cast<int64_t>(kvh) * kPage * d;
  const int off = slot % kPage;
  for (int i = threadIdx.x; i < d; i += kWave) {
    float ks = 0.f, vs = 0.f;
    int j = pos - block + 1;
    for (; j + 3 <= pos; j += 4) {                       // four positions' loads in flight, added in the positions' order
      float kq[4], vq[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const A* src = kv + static_cast<int64_t>(table[(j + q) / kPage]) * page_elems + static_cast<int64_t>(kvh) * kPage * d;
        kq[q] = to_float<A>(src[((j + q) % kPage) * d + i]);
        vq[q] = to_float<A>(src[half + static_cast<int64_t>(i) * kPage + ((j + q) % kPage)]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        ks += kq[q];
        vs += vq[q];
      }
    }
    for (; j <= pos; ++j) {
      const A* src = kv + static_cast<int64_t>(table[j / kPage]) * page_elems + static_cast<int64_t>(kvh) * kPage * d;
      ks += to_float<A>(src[(j % kPage) * d + i]);
      vs += to_float<A>(src[half + static_cast<int64_t>(i) * kPage + (j % kPage)]);
    }
    dst[off * d + i] = from_float<A>(ks * inv);
    dst[half + static_cast<int64_t>(i) * kPage + off] = from_float<A>(vs * inv);
  }
}

}  // namespace psamd

using namespace psamd;

#define PSAMD_BY_DTYPE(code, CALL)                                                   \
  if ((code) == kBF16) { using A_ = bf16_t; CALL; }                                  \
  else if ((code) == kF32) { using A_ = float; CALL; }                               \
  else return fail(std::string(__func__) + ": dtype must be float32 or bfloat16")

extern "C" {

int psamd_stream_rms_norm(void* stream, float* x, const float* weight, float eps, int64_t rows, int hidden) {
  PSAMD_REQUIRE(rows >= 0 && rows <= 2147483647LL && hidden > 0, "bad sizes");
  if (rows == 0) return 0;
  stream_rms_norm_kernel<<<dim3(static_cast<unsigned>(rows)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, weight, eps, hidden);
  return check_launch("psamd_stream_rms_norm");
}

int psamd_hyper_read(void* stream, const float* streams, int count, const float* read, const float* weight, float eps,
                     const float* factor, void* out, int out_dtype, int64_t tokens, int hidden) {
  PSAMD_REQUIRE(tokens >= 0 && tokens <= 2147483647LL && hidden > 0 && count >= 1 && count <= kMaxStreams, "bad sizes (at most 16 streams)");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t stride = tokens * hidden;
  const size_t smem = sizeof(float) * static_cast<size_t>(hidden);
  PSAMD_REQUIRE(smem <= 60 * 1024, "rows of up to 15,360 numbers");
#define PSAMD_READ(C_)                                                                                                   \
  PSAMD_BY_DTYPE(out_dtype, (hyper_read_kernel<A_, C_><<<dim3(static_cast<unsigned>(tokens)), dim3(256), smem, s>>>(     \
                                streams, stride, count, read, weight, eps, factor, static_cast<A_*>(out), hidden)))
  switch (count) {
    case 1: PSAMD_READ(1); break;
    case 2: PSAMD_READ(2); break;
    case 3: PSAMD_READ(3); break;
    case 4: PSAMD_READ(4); break;
    case 8: PSAMD_READ(8); break;
    default: PSAMD_READ(0); break;
  }
#undef PSAMD_READ
  return check_launch("psamd_hyper_read");
}

int psamd_hyper_write(void* stream, float* streams, int count, const float* mix, const float* write, const void* a,
                      int a_dtype, int a_slices, int64_t a_stride, float a_scale, const void* b, int b_dtype, int b_slices,
                      int64_t b_stride, float b_scale, int64_t tokens, int hidden) {
  PSAMD_REQUIRE(tokens >= 0 && hidden > 0 && count >= 1 && count <= kMaxStreams && a_slices >= 1 && b_slices >= 1,
                "bad sizes (at most 16 streams)");
  PSAMD_REQUIRE((a_dtype == kF32 || (a_dtype == kBF16 && a_slices == 1)) && (b == nullptr || b_dtype == kF32 || (b_dtype == kBF16 && b_slices == 1)),
                "an output is one tensor or float slices");
  const int64_t n = tokens * hidden;
  if (n == 0) return 0;
  PSAMD_REQUIRE(ceil_div(n, 256) <= 2147483647LL, "too large for one launch");
  hyper_write_kernel<<<dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      streams, n, count, mix, write, a, a_dtype, a_slices, a_stride, a_scale, b, b_dtype, b_slices, b_stride, b_scale, n);
  return check_launch("psamd_hyper_write");
}

int psamd_weighted_sum(void* stream, const void* a, int a_dtype, int a_slices, int64_t a_stride, float a_scale, const void* b,
                       int b_dtype, int b_slices, int64_t b_stride, float b_scale, float* out, int64_t n) {
  PSAMD_REQUIRE(n >= 0 && a_slices >= 1 && b_slices >= 1, "bad sizes");
  PSAMD_REQUIRE((a_dtype == kF32 || (a_dtype == kBF16 && a_slices == 1)) && (b_dtype == kF32 || (b_dtype == kBF16 && b_slices == 1)),
                "an operand is one tensor or float slices");
  if (n == 0) return 0;
  PSAMD_REQUIRE(ceil_div(n, 256) <= 2147483647LL, "too large for one launch");
  weighted_sum_kernel<<<dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      a, a_dtype, a_slices, a_stride, a_scale, b, b_dtype, b_slices, b_stride, b_scale, out, n);
  return check_launch("psamd_weighted_sum");
}

int psamd_activation(void* stream, void* x, int act_dtype, int64_t n, int kind) {
  PSAMD_REQUIRE(n >= 0 && kind >= 0 && kind <= 3, "bad size or activation");
  if (n == 0) return 0;
  PSAMD_REQUIRE(ceil_div(n, 256) <= 2147483647LL, "too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  PSAMD_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0, "the tensor must start at a multiple of 16 bytes");
  const int64_t threads = n / (act_dtype == kBF16 ? 8 : 4) + 1;
  PSAMD_BY_DTYPE(act_dtype, (activation_kernel<A_><<<dim3(static_cast<unsigned>(ceil_div(threads, 256))), dim3(256), 0, s>>>(
                                static_cast<A_*>(x), n, kind)));
  return check_launch("psamd_activation");
}

int psamd_gated_group_norm(void* stream, const float* y, const float* x, int64_t x_row, const float* skip, int heads,
                           const void* gate, int act_dtype, int64_t gate_row, const float* weight, int parts, float eps,
                           void* out, int64_t tokens, int inner) {
  PSAMD_REQUIRE(tokens >= 0 && inner > 0 && heads > 0 && parts > 0 && inner % heads == 0 && inner % parts == 0, "bad sizes");
  const int64_t pairs = tokens * parts;
  if (pairs == 0) return 0;
  PSAMD_REQUIRE(ceil_div(pairs, 4) <= 2147483647LL, "too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (inner / parts > 256) {
    PSAMD_REQUIRE(pairs <= 2147483647LL, "too large for one launch");
    PSAMD_BY_DTYPE(act_dtype, (gated_group_norm_kernel<A_, 4><<<dim3(static_cast<unsigned>(pairs)), dim3(256), 0, s>>>(
                                  y, x, x_row, skip, inner / heads, static_cast<const A_*>(gate), gate_row, weight, parts,
                                  inner / parts, eps, static_cast<A_*>(out), pairs)));
  } else {
    PSAMD_BY_DTYPE(act_dtype, (gated_group_norm_kernel<A_, 1><<<dim3(static_cast<unsigned>(ceil_div(pairs, 4))), dim3(256), 0, s>>>(
                                  y, x, x_row, skip, inner / heads, static_cast<const A_*>(gate), gate_row, weight, parts,
                                  inner / parts, eps, static_cast<A_*>(out), pairs)));
  }
  return check_launch("psamd_gated_group_norm");
}

int psamd_state_space_prepare(void* stream, const float* dt, const float* dt_bias, const float* a_log, float* coef,
                              int64_t tokens, int heads) {
  PSAMD_REQUIRE(tokens >= 0 && heads > 0, "bad sizes");
  const int64_t n = tokens * heads;
  if (n == 0) return 0;
  state_space_prepare_kernel<<<dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      dt, dt_bias, a_log, coef, n, heads);
  return check_launch("psamd_state_space_prepare");
}

int psamd_matrix_memory_gates(void* stream, const float* gates, const float* bias, float cap, float* coef, float* state,
                              int64_t state_row, const int32_t* item_start, const int32_t* slots, int items, int heads) {
  PSAMD_REQUIRE(items >= 0 && heads > 0 && cap > 0.f && state_row >= heads, "bad sizes");
  if (items == 0) return 0;
  PSAMD_REQUIRE(heads <= 65535, "too many heads for one launch");
  matrix_memory_gates_kernel<<<dim3(static_cast<unsigned>(items), static_cast<unsigned>(heads)), dim3(64), 0,
                               static_cast<hipStream_t>(stream)>>>(
      gates, bias, cap, coef, state, state_row, item_start, slots, heads);
  return check_launch("psamd_matrix_memory_gates");
}

int psamd_matrix_memory_operands(void* stream, const void* rows, int act_dtype, int64_t in_row, int q_col, int k_col, int v_col,
                                 int heads, int dim, int vdim, float q_scale, float* u, float* vals, int64_t tokens) {
  PSAMD_REQUIRE(tokens >= 0 && tokens <= 2147483647LL && heads > 0 && dim > 0 && vdim > 0, "bad sizes");
  PSAMD_REQUIRE(std::min(std::min(q_col, k_col), v_col) >= 0 && std::max(q_col, k_col) + static_cast<int64_t>(heads) * dim <= in_row &&
                    v_col + static_cast<int64_t>(heads) * vdim <= in_row, "columns outside the rows");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  PSAMD_BY_DTYPE(act_dtype, (matrix_memory_operands_kernel<A_><<<dim3(static_cast<unsigned>(tokens)), dim3(256), 0, s>>>(
                                static_cast<const A_*>(rows), in_row, q_col, k_col, v_col, heads, dim, vdim, q_scale, u, vals)));
  return check_launch("psamd_matrix_memory_operands");
}

int psamd_memory_read_norm_gate(void* stream, const float* raw, const float* floor_, int64_t floor_row, int heads, int vdim,
                                float read_eps, const float* weight, float eps, const void* gate, int act_dtype,
                                int64_t gate_row, void* out, int64_t tokens) {
  PSAMD_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0, "bad sizes");
  const int64_t pairs = tokens * heads;
  if (pairs == 0) return 0;
  PSAMD_REQUIRE(ceil_div(pairs, 4) <= 2147483647LL, "too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  PSAMD_BY_DTYPE(act_dtype, (memory_read_norm_gate_kernel<A_><<<dim3(static_cast<unsigned>(ceil_div(pairs, 4))), dim3(256), 0, s>>>(
                                raw, floor_, floor_row, heads, vdim, read_eps, weight, eps, static_cast<const A_*>(gate),
                                gate_row, static_cast<A_*>(out), pairs)));
  return check_launch("psamd_memory_read_norm_gate");
}

int psamd_pool_kv_append(void* stream, const void* kv, void* pool, int act_dtype, const int32_t* positions,
                         const int32_t* tok_item, const int32_t* table_off, const int32_t* block_ids, const int32_t* pool_slot,
                         int64_t tokens, int hkv, int head_dim, int block) {
  PSAMD_REQUIRE(tokens >= 0 && tokens <= 2147483647LL && hkv > 0 && hkv <= 65535 && head_dim > 0 && block >= 1, "bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(hkv));
  PSAMD_BY_DTYPE(act_dtype, (pool_kv_append_kernel<A_><<<grid, dim3(64), 0, s>>>(
                                static_cast<const A_*>(kv), static_cast<A_*>(pool), positions, tok_item, table_off, block_ids,
                                pool_slot, hkv, head_dim, block)));
  return check_launch("psamd_pool_kv_append");
}

}  // extern "C"
