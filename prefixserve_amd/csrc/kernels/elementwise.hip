// Memory-bound kernels around the matrix products: token gather, fused residual-add +
// RMSNorm, SwiGLU, and rotary encoding fused with the write of keys and values into their
// cache pages. Each is templated on the activation type (bfloat16 or float); statistics,
// rotation and the residual sum are always float.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

static thread_local std::string g_error;
void set_error(const std::string& msg) { g_error = msg; }

// ------------------------------------------------------------------ embed

template <typename W>
__global__ void embed_kernel(const int32_t* __restrict__ ids, const W* __restrict__ table,
                             float* __restrict__ out, int hidden, int vocab) {
  const int64_t t = blockIdx.x;
  // Ids are checked on the host, except those a previous step sampled and left on the device:
  // an id outside the table reads its nearest row instead of memory that is not the table's.
  const int id = min(max(ids[t], 0), vocab - 1);
  const W* row = table + static_cast<int64_t>(id) * hidden;
  float* o = out + t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = to_float<W>(row[i]);
}

// ------------------------------------------------------------------ add + rmsnorm

// One block per output row. x = residual + sum of the delta slices; out = weight * x *
// rsqrt(mean(x^2) + eps), everything in float. `delta` is either [rows, hidden] in the
// activation type or n_partials float slices [n_partials][rows, hidden] (partial sums of a
// K-split product). Without `rows` the block handles row blockIdx.x and stores x back as the
// new residual; with `rows` it handles residual row rows[blockIdx.x] and leaves it as it is.
// Rows up to kCache * kThreads wide stay in registers between the two passes, and all loads
// of a pass are independent of each other (clamped addresses, no branches around them), so
// they are in flight together: with one row per block the kernel is pure latency.
template <typename A, typename DT, int kThreads, int kCache>
__global__ __launch_bounds__(kThreads) void add_rmsnorm_kernel(
    float* __restrict__ residual, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const int32_t* __restrict__ rows, const void* __restrict__ weight, int weight_dtype, float eps,
    A* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  const int64_t src = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  float* r = residual + src * hidden;
  const DT* d0 = delta != nullptr ? delta + src * hidden : nullptr;
  A* o = out + static_cast<int64_t>(blockIdx.x) * hidden;
  const bool store = rows == nullptr && delta != nullptr;
  const int np = delta != nullptr ? n_partials : 0;

  if (hidden <= kCache * kThreads) {
    float v[kCache], wv[kCache];
    int idx[kCache];
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      idx[j] = min(static_cast<int>(threadIdx.x) + j * kThreads, hidden - 1);
      v[j] = r[idx[j]];
      wv[j] = load_as_float(weight, weight_dtype, idx[j]);
    }
    for (int p = 0; p < np; ++p) {
      const DT* dp = d0 + p * partial_stride;
      float t[kCache];
#pragma unroll
      for (int j = 0; j < kCache; ++j) t[j] = to_float<DT>(dp[idx[j]]);
#pragma unroll
      for (int j = 0; j < kCache; ++j) v[j] += t[j];
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      const bool in = static_cast<int>(threadIdx.x) + j * kThreads < hidden;
      ss += in ? v[j] * v[j] : 0.f;
    }
    ss = block_sum(ss, scratch, kThreads / kWave);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      if (static_cast<int>(threadIdx.x) + j * kThreads < hidden) {
        if (store) r[idx[j]] = v[j];
        o[idx[j]] = from_float<A>(wv[j] * (v[j] * inv));
      }
    }
    return;
  }

  auto value = [&](int i) {
    float x = r[i];
    for (int p = 0; p < np; ++p) x += to_float<DT>(d0[p * partial_stride + i]);
    return x;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = value(i);
    if (store) r[i] = x;
    ss += x * x;
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float x = store ? r[i] : value(i);
    o[i] = from_float<A>(load_as_float(weight, weight_dtype, i) * (x * inv));
  }
}

// The same operation for bfloat16 activations and rows that are a multiple of 8 wide: every
// thread owns runs of 8 consecutive elements, moved as 16- and 32-byte accesses. kIter runs
// per thread stay in registers (hidden <= 8 * kThreads * kIter).
template <typename DT, int kThreads, int kIter>
__global__ __launch_bounds__(kThreads) void add_rmsnorm_vec8_kernel(
    float* __restrict__ residual, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const int32_t* __restrict__ rows, const void* __restrict__ weight, int weight_dtype, float eps,
    bf16_t* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  const int64_t src = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  float* r = residual + src * hidden;
  const DT* d0 = delta != nullptr ? delta + src * hidden : nullptr;
  bf16_t* o = out + static_cast<int64_t>(blockIdx.x) * hidden;
  const bool store = rows == nullptr && delta != nullptr;
  const int np = delta != nullptr ? n_partials : 0;
  const int chunks = hidden >> 3;

  float v[kIter][8];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = threadIdx.x + j * kThreads;
    const int e = min(cidx, chunks - 1) << 3;
    const float4 a = *reinterpret_cast<const float4*>(r + e);
    const float4 b = *reinterpret_cast<const float4*>(r + e + 4);
    v[j][0] = a.x; v[j][1] = a.y; v[j][2] = a.z; v[j][3] = a.w;
    v[j][4] = b.x; v[j][5] = b.y; v[j][6] = b.z; v[j][7] = b.w;
    for (int p = 0; p < np; ++p) {
      const DT* dp = d0 + p * partial_stride + e;
      if (sizeof(DT) == 2) {
        const uint4 q = *reinterpret_cast<const uint4*>(dp);
        const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[j][2 * i] += __uint_as_float(w4[i] << 16);
          v[j][2 * i + 1] += __uint_as_float(w4[i] & 0xffff0000u);
        }
      } else {
        // Up to eight slices are asked for together (one trip to memory, not one per slice) and
        // added in ascending order; slots past the last slice repeat it and are not added.
        float4 x0[8], x1[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const DT* du = d0 + min(p + u, np - 1) * partial_stride + e;
          x0[u] = *reinterpret_cast<const float4*>(du);
          x1[u] = *reinterpret_cast<const float4*>(du + 4);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (p + u < np) {
            v[j][0] += x0[u].x; v[j][1] += x0[u].y; v[j][2] += x0[u].z; v[j][3] += x0[u].w;
            v[j][4] += x1[u].x; v[j][5] += x1[u].y; v[j][6] += x1[u].z; v[j][7] += x1[u].w;
          }
        }
        p += 7;
      }
    }
    if (cidx < chunks) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[j][i] * v[j][i];
    }
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = threadIdx.x + j * kThreads;
    if (cidx >= chunks) continue;
    const int e = cidx << 3;
    if (store) {
      *reinterpret_cast<float4*>(r + e) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
      *reinterpret_cast<float4*>(r + e + 4) = make_float4(v[j][4], v[j][5], v[j][6], v[j][7]);
    }
    float w[8];
    if (weight_dtype == kBF16) {
      const uint4 q = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(weight) + e);
      const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        w[2 * i] = __uint_as_float(w4[i] << 16);
        w[2 * i + 1] = __uint_as_float(w4[i] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) w[i] = static_cast<const float*>(weight)[e + i];
    }
    uint32_t pk[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pk[i] = static_cast<uint32_t>(float_to_bf16(w[2 * i] * (v[j][2 * i] * inv))) |
              (static_cast<uint32_t>(float_to_bf16(w[2 * i + 1] * (v[j][2 * i + 1] * inv))) << 16);
    }
    *reinterpret_cast<uint4*>(o + e) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

// ------------------------------------------------------------------ swiglu

template <typename A>
__global__ void swiglu_kernel(const A* __restrict__ gate_up, A* __restrict__ out, int64_t tokens, int inter, int act) {
  const int64_t n = tokens * inter;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / inter, c = i - t * inter;
    const float g = to_float<A>(gate_up[t * 2 * inter + c]);
    const float u = to_float<A>(gate_up[t * 2 * inter + inter + c]);
    out[i] = from_float<A>(gate_act(g, act) * u);
  }
}

// bfloat16, intermediate size a multiple of 8: 16-byte accesses, 8 elements per thread.
__global__ void swiglu_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int64_t tokens,
                                   int inter, int act) {
  const int chunks = inter >> 3;
  const int64_t n = tokens * chunks;
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = i / chunks;
    const int e = static_cast<int>(i - t * chunks) << 3;
    const uint4 g = *reinterpret_cast<const uint4*>(gate_up + t * 2 * inter + e);
    const uint4 u = *reinterpret_cast<const uint4*>(gate_up + t * 2 * inter + inter + e);
    const uint32_t g4[4] = {g.x, g.y, g.z, g.w}, u4[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g0 = __uint_as_float(g4[k] << 16), g1 = __uint_as_float(g4[k] & 0xffff0000u);
      const float u0 = __uint_as_float(u4[k] << 16), u1 = __uint_as_float(u4[k] & 0xffff0000u);
      pk[k] = static_cast<uint32_t>(float_to_bf16(gate_act(g0, act) * u0)) |
              (static_cast<uint32_t>(float_to_bf16(gate_act(g1, act) * u1)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * inter + e) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
  }
}

// ------------------------------------------------------------------ rope + kv append

// One block per token. q and k heads of the fused qkv row are rotated in place (pair
// (i, i + D/2), angle table [pos][i] = (cos, sin)); the rotated keys go to their page as
// [16, D] rows and the values to the page's second half transposed, [D, 16].
template <typename A>
__global__ void rope_kv_append_kernel(A* __restrict__ qkv, int hq, int hkv, int d,
                                      const int32_t* __restrict__ positions,
                                      const float2* __restrict__ table,
                                      A* __restrict__ kv, const int32_t* __restrict__ write_slot) {
  const int64_t t = blockIdx.x;
  const int half = d / 2;
  A* row = qkv + t * static_cast<int64_t>((hq + 2 * hkv) * d);
  const int pos = positions[t];
  int64_t page = 0;
  int off = 0;
  if (kv != nullptr) {
    const int slot = write_slot[t];
    page = slot / kPage;
    off = slot % kPage;
  }
  const int64_t page_elems = 2LL * hkv * kPage * d;
  A* kpage = kv != nullptr ? kv + page * page_elems : nullptr;
  A* vpage = kv != nullptr ? kpage + static_cast<int64_t>(hkv) * kPage * d : nullptr;

  const int n_rot = (hq + hkv) * half;
  for (int idx = threadIdx.x; idx < n_rot; idx += blockDim.x) {
    const int h = idx / half, i = idx - h * half;
    A* x = row + h * d;
    float a = to_float<A>(x[i]), b = to_float<A>(x[i + half]);
    if (table != nullptr) {
      const float2 cs = table[static_cast<int64_t>(pos) * half + i];
      const float ra = a * cs.x - b * cs.y;
      const float rb = b * cs.x + a * cs.y;
      a = ra;
      b = rb;
      x[i] = from_float<A>(a);
      x[i + half] = from_float<A>(b);
    }
    if (kpage != nullptr && h >= hq) {
      A* dst = kpage + (static_cast<int64_t>(h - hq) * kPage + off) * d;
      dst[i] = from_float<A>(a);
      dst[i + half] = from_float<A>(b);
    }
  }
  if (vpage != nullptr) {
    const A* v = row + (hq + hkv) * d;
    for (int idx = threadIdx.x; idx < hkv * d; idx += blockDim.x) {
      const int h = idx / d, c = idx - h * d;
      vpage[(static_cast<int64_t>(h) * d + c) * kPage + off] = v[idx];
    }
  }
}

// bfloat16 with a head size that is a multiple of 16: one block per 16 tokens of the step.
// q and k are rotated eight pairs per thread with 16-byte accesses. The values of the 16
// tokens pass through LDS so that lanes 0..15 write the same (head, dim) of 16 tokens: when
// the tokens follow each other in one page, as the tokens of a prompt do, that is one 32-byte
// run of the transposed page instead of 16 scattered 2-byte stores.
__global__ __launch_bounds__(256) void rope_kv_append_vec_kernel(bf16_t* __restrict__ qkv, int tokens, int hq, int hkv,
                                                                 int d, const int32_t* __restrict__ positions,
                                                                 const float2* __restrict__ table,
                                                                 bf16_t* __restrict__ kv,
                                                                 const int32_t* __restrict__ write_slot) {
  extern __shared__ __align__(16) bf16_t v_lds[];        // [16][hkv * d + 8]
  const int t0 = blockIdx.x * 16;
  const int nt = min(16, tokens - t0);
  const int half = d >> 1;
  const int width = (hq + 2 * hkv) * d;
  const int64_t page_elems = 2LL * hkv * kPage * d;
  const int chunks_per_head = half >> 3;                 // groups of 8 pairs
  const int chunks_per_token = (hq + hkv) * chunks_per_head;
  const int vw = hkv * d;
  const int c_lo = static_cast<int>(static_cast<int64_t>(vw >> 3) * blockIdx.y / gridDim.y);      // 8-element columns
  const int c_hi = static_cast<int>(static_cast<int64_t>(vw >> 3) * (blockIdx.y + 1) / gridDim.y);
  const int nc = c_hi - c_lo, vs = 8 * nc + 8;
  // The values are asked for first: they are on their way into LDS while q and k are rotated.
  for (int idx = threadIdx.x; kv != nullptr && idx < nt * nc; idx += blockDim.x) {
    const int j = idx / nc, c = idx - j * nc;
    *reinterpret_cast<uint4*>(v_lds + j * vs + 8 * c) =
        *reinterpret_cast<const uint4*>(qkv + static_cast<int64_t>(t0 + j) * width + (hq + hkv) * d + 8 * (c_lo + c));
  }
  // blockIdx.y takes its share of the rotation work and of the value columns.
  const int rot_total = nt * chunks_per_token;
  const int rot_lo = static_cast<int>(static_cast<int64_t>(rot_total) * blockIdx.y / gridDim.y);
  const int rot_hi = static_cast<int>(static_cast<int64_t>(rot_total) * (blockIdx.y + 1) / gridDim.y);
  for (int idx = rot_lo + threadIdx.x; idx < rot_hi; idx += blockDim.x) {
    const int j = idx / chunks_per_token, c = idx - j * chunks_per_token;
    const int h = c / chunks_per_head, i = (c - h * chunks_per_head) << 3;
    const int64_t t = t0 + j;
    bf16_t* x = qkv + t * width + h * d + i;
    uint4 lo = *reinterpret_cast<const uint4*>(x), hi = *reinterpret_cast<const uint4*>(x + half);
    if (table != nullptr) {
      const float2* cs = table + static_cast<int64_t>(positions[t]) * half + i;
      const uint32_t* lw = reinterpret_cast<const uint32_t*>(&lo);
      const uint32_t* hw = reinterpret_cast<const uint32_t*>(&hi);
      uint32_t lo_out[4], hi_out[4];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float a0 = bf16_to_float(static_cast<bf16_t>(lw[w] & 0xffffu)), a1 = bf16_to_float(static_cast<bf16_t>(lw[w] >> 16));
        const float b0 = bf16_to_float(static_cast<bf16_t>(hw[w] & 0xffffu)), b1 = bf16_to_float(static_cast<bf16_t>(hw[w] >> 16));
        const float2 c0 = cs[2 * w], c1 = cs[2 * w + 1];
        lo_out[w] = static_cast<uint32_t>(float_to_bf16(a0 * c0.x - b0 * c0.y)) |
                    (static_cast<uint32_t>(float_to_bf16(a1 * c1.x - b1 * c1.y)) << 16);
        hi_out[w] = static_cast<uint32_t>(float_to_bf16(b0 * c0.x + a0 * c0.y)) |
                    (static_cast<uint32_t>(float_to_bf16(b1 * c1.x + a1 * c1.y)) << 16);
      }
      lo = make_uint4(lo_out[0], lo_out[1], lo_out[2], lo_out[3]);
      hi = make_uint4(hi_out[0], hi_out[1], hi_out[2], hi_out[3]);
      *reinterpret_cast<uint4*>(x) = lo;
      *reinterpret_cast<uint4*>(x + half) = hi;
    }
    if (kv != nullptr && h >= hq) {
      const int slot = write_slot[t];
      bf16_t* dst = kv + static_cast<int64_t>(slot / kPage) * page_elems +
                    (static_cast<int64_t>(h - hq) * kPage + slot % kPage) * d + i;
      *reinterpret_cast<uint4*>(dst) = lo;
      *reinterpret_cast<uint4*>(dst + half) = hi;
    }
  }
  if (kv == nullptr) return;
  __syncthreads();
  const int j = threadIdx.x & 15;
  if (j < nt) {
    const int slot = write_slot[t0 + j];
    bf16_t* vpage = kv + static_cast<int64_t>(slot / kPage) * page_elems + static_cast<int64_t>(hkv) * kPage * d + slot % kPage;
    for (int e = threadIdx.x >> 4; e < 8 * nc; e += blockDim.x >> 4)
      vpage[static_cast<int64_t>(8 * c_lo + e) * kPage] = v_lds[j * vs + e];
  }
}

// ------------------------------------------------------------------ norm behind the sum

// One block per row: x = alpha * residual + sum of the delta slices, y = weight * x *
// rsqrt(mean(x^2) + eps), all in float; y becomes the new residual row and, if `out` is given,
// is also written in the activation type (the copy the next product reads). Rows up to
// kCache * kThreads wide stay in registers between the two passes; wider ones pass through
// the residual row itself.
template <typename A, typename DT, int kThreads, int kCache>
__global__ __launch_bounds__(kThreads) void scaled_add_rmsnorm_kernel(
    float* __restrict__ residual, float alpha, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const void* __restrict__ weight, int weight_dtype, float eps, A* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  float* r = residual + static_cast<int64_t>(blockIdx.x) * hidden;
  const DT* d0 = delta != nullptr ? delta + static_cast<int64_t>(blockIdx.x) * hidden : nullptr;
  A* o = out != nullptr ? out + static_cast<int64_t>(blockIdx.x) * hidden : nullptr;
  const int np = delta != nullptr ? n_partials : 0;
  if (hidden <= kCache * kThreads) {
    float v[kCache];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      const int i = static_cast<int>(threadIdx.x) + j * kThreads;
      const int ic = min(i, hidden - 1);
      float x = alpha * r[ic];
      for (int p = 0; p < np; ++p) x += to_float<DT>(d0[p * partial_stride + ic]);
      v[j] = x;
      ss += i < hidden ? x * x : 0.f;
    }
    ss = block_sum(ss, scratch, kThreads / kWave);
    const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int j = 0; j < kCache; ++j) {
      const int i = static_cast<int>(threadIdx.x) + j * kThreads;
      if (i < hidden) {
        const float y = load_as_float(weight, weight_dtype, i) * (v[j] * inv);
        r[i] = y;
        if (o != nullptr) o[i] = from_float<A>(y);
      }
    }
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    float x = alpha * r[i];
    for (int p = 0; p < np; ++p) x += to_float<DT>(d0[p * partial_stride + i]);
    r[i] = x;
    ss += x * x;
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kThreads) {
    const float y = load_as_float(weight, weight_dtype, i) * (r[i] * inv);
    r[i] = y;
    if (o != nullptr) o[i] = from_float<A>(y);
  }
}

// The same for rows that are a multiple of 4 wide, up to 4 * kThreads * kIter: every thread owns
// runs of 4 consecutive elements (16-byte accesses of the stream and of float slices), and up to
// four slices are asked for together and added in ascending order.
template <typename A, typename DT, int kThreads, int kIter>
__global__ __launch_bounds__(kThreads) void scaled_add_rmsnorm_vec4_kernel(
    float* __restrict__ residual, float alpha, const DT* __restrict__ delta, int n_partials, int64_t partial_stride,
    const void* __restrict__ weight, int weight_dtype, float eps, A* __restrict__ out, int hidden) {
  __shared__ float scratch[kThreads / kWave];
  float* r = residual + static_cast<int64_t>(blockIdx.x) * hidden;
  const DT* d0 = delta != nullptr ? delta + static_cast<int64_t>(blockIdx.x) * hidden : nullptr;
  A* o = out != nullptr ? out + static_cast<int64_t>(blockIdx.x) * hidden : nullptr;
  const int np = delta != nullptr ? n_partials : 0;
  const int chunks = hidden >> 2;
  float4 v[kIter];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = static_cast<int>(threadIdx.x) + j * kThreads;
    const int e = min(cidx, chunks - 1) << 2;
    float4 x = *reinterpret_cast<const float4*>(r + e);
    x.x *= alpha; x.y *= alpha; x.z *= alpha; x.w *= alpha;
    if (sizeof(DT) == 2) {
      if (np > 0) {
        const uint2 q = *reinterpret_cast<const uint2*>(d0 + e);
        x.x += __uint_as_float(q.x << 16); x.y += __uint_as_float(q.x & 0xffff0000u);
        x.z += __uint_as_float(q.y << 16); x.w += __uint_as_float(q.y & 0xffff0000u);
      }
    } else {
      for (int p = 0; p < np; p += 4) {
        float4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          t[u] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(d0) + min(p + u, np - 1) * partial_stride + e);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (p + u < np) { x.x += t[u].x; x.y += t[u].y; x.z += t[u].z; x.w += t[u].w; }
        }
      }
    }
    v[j] = x;
    if (cidx < chunks) ss += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
  }
  ss = block_sum(ss, scratch, kThreads / kWave);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
#pragma unroll
  for (int j = 0; j < kIter; ++j) {
    const int cidx = static_cast<int>(threadIdx.x) + j * kThreads;
    if (cidx >= chunks) continue;
    const int e = cidx << 2;
    float4 y;
    y.x = load_as_float(weight, weight_dtype, e) * (v[j].x * inv);
    y.y = load_as_float(weight, weight_dtype, e + 1) * (v[j].y * inv);
    y.z = load_as_float(weight, weight_dtype, e + 2) * (v[j].z * inv);
    y.w = load_as_float(weight, weight_dtype, e + 3) * (v[j].w * inv);
    *reinterpret_cast<float4*>(r + e) = y;
    if (o != nullptr) {
      if (sizeof(A) == 2) {
        ushort4 pk;
        pk.x = float_to_bf16(y.x); pk.y = float_to_bf16(y.y); pk.z = float_to_bf16(y.z); pk.w = float_to_bf16(y.w);
        *reinterpret_cast<ushort4*>(reinterpret_cast<bf16_t*>(o) + e) = pk;
      } else {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(o) + e) = y;
      }
    }
  }
}

// out[i] = A(in[i]): the float32 stream in the activation type.
template <typename A>
__global__ void to_activation_kernel(const float* __restrict__ in, A* __restrict__ out, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    out[i] = from_float<A>(in[i]);
}

// ------------------------------------------------------------------ rope + unit norm + kv append

// A group of L lanes per (token, head) of a row [hq q heads | hkv k heads | hkv v heads] x d, L the
// power of two that holds d/2 pairs (at most a wave: several heads share a wave when d < 128). A q
// or k head is rotated (pair (i, i + d/2), table [pos][i] = (cos, sin); NULL: not rotated), then, with
// norm_dim > 0, divided by sqrt(sum of squares / norm_dim + eps): the root mean square over the
// norm_dim dimensions that are the head's own when the rest of its d slots hold zeros. The
// result goes back into the row and, for a k head, to its page as a [16, d] row; a v head goes
// to the page's second half transposed, [d, 16]. hkv may be 0 (a row of queries alone).
template <typename A>
__global__ __launch_bounds__(256) void rope_norm_kv_append_kernel(
    A* __restrict__ qkv, int hq, int hkv, int d, const int32_t* __restrict__ positions,
    const float2* __restrict__ table, int norm_dim, float eps, A* __restrict__ kv,
    const int32_t* __restrict__ write_slot, int group_lanes, const float* __restrict__ bias,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, int v_from_k, int q_weight_stride) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int per_wave = kWave / group_lanes;
  const int l = lane & (group_lanes - 1);
  const int head = (static_cast<int>(blockIdx.y) * 4 + static_cast<int>(threadIdx.x >> 6)) * per_wave + lane / group_lanes;
  const int row_heads = hq + (v_from_k ? hkv : 2 * hkv);
  if (head >= row_heads) return;
  const int half = d >> 1;
  A* row = qkv + t * (static_cast<int64_t>(row_heads) * d) + static_cast<int64_t>(head) * d;
  int64_t page = 0;
  int off = 0;
  if (kv != nullptr) {
    const int slot = write_slot[t];
    page = slot / kPage;
    off = slot % kPage;
  }
  const int64_t page_elems = 2LL * hkv * kPage * d;
  if (head < hq + hkv) {
    const int pos = positions[t];
    // q_weight_stride = d: every query head has a weight of its own (a number per head folded into it)
    const float* nw = head < hq ? (q_weight != nullptr ? q_weight + static_cast<int64_t>(head) * q_weight_stride : nullptr) : k_weight;
    float a[2], b[2];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {                      // group_lanes = 64 when d > 128: two pairs per lane
      const int i = l + j * group_lanes;
      a[j] = b[j] = 0.f;
      if (i < half) {
        float u = to_float<A>(row[i]), v = to_float<A>(row[i + half]);
        if (bias != nullptr) {
          u += bias[static_cast<int64_t>(head) * d + i];
          v += bias[static_cast<int64_t>(head) * d + i + half];
        }
        if (v_from_k && head >= hq && kv != nullptr) {
          // the value is the key as projected: before rotation and norm
          A* vpage = kv + page * page_elems + static_cast<int64_t>(hkv) * kPage * d + off;
          vpage[(static_cast<int64_t>(head - hq) * d + i) * kPage] = from_float<A>(u);
          vpage[(static_cast<int64_t>(head - hq) * d + i + half) * kPage] = from_float<A>(v);
        }
        float2 cs = float2{1.f, 0.f};
        if (table != nullptr) cs = table[static_cast<int64_t>(pos) * half + i];
        a[j] = u * cs.x - v * cs.y;
        b[j] = v * cs.x + u * cs.y;
        ss += a[j] * a[j] + b[j] * b[j];
      }
    }
    float inv = 1.f;
    if (norm_dim > 0) {
      // the sum over the head's group of lanes: partners of every step lie inside the group
      for (int o = group_lanes >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
      inv = rsqrtf(ss / static_cast<float>(norm_dim) + eps);
    }
    A* dst = (kv != nullptr && head >= hq)
                 ? kv + page * page_elems + (static_cast<int64_t>(head - hq) * kPage + off) * d : nullptr;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = l + j * group_lanes;
      if (i < half) {
        const A lo = from_float<A>(a[j] * inv * (nw != nullptr ? nw[i] : 1.f));
        const A hi = from_float<A>(b[j] * inv * (nw != nullptr ? nw[i + half] : 1.f));
        row[i] = lo;
        row[i + half] = hi;
        if (dst != nullptr) {
          dst[i] = lo;
          dst[i + half] = hi;
        }
      }
    }
  } else if (kv != nullptr) {
    const int vh = head - hq - hkv;
    A* vpage = kv + page * page_elems + static_cast<int64_t>(hkv) * kPage * d + off;
    for (int c = l; c < d; c += group_lanes) vpage[(static_cast<int64_t>(vh) * d + c) * kPage] = row[c];
  }
}

// ------------------------------------------------------------------ sums and copies of the stream

// residual += delta, where delta is one tensor or n_partials float32 slices (summed in ascending order).
template <typename DT>
__global__ void residual_add_kernel(float* __restrict__ residual, const DT* __restrict__ delta, int n_partials,
                                    int64_t partial_stride, int64_t n) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    float x = residual[i];
    for (int p = 0; p < n_partials; ++p) x += to_float<DT>(delta[p * partial_stride + i]);
    residual[i] = x;
  }
}

__global__ void stream_affine_kernel(float* __restrict__ x, int64_t n, int hidden, float factor,
                                     const float* __restrict__ row) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const float add = row != nullptr ? row[i % hidden] : 0.f;
    x[i] = x[i] * factor + add;
  }
}

template <typename A>
__global__ void concat_to_activation_kernel(const float* __restrict__ a, const float* __restrict__ b, A* __restrict__ out,
                                            int64_t n, int hidden) {
  for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = i / hidden, c = i - r * hidden;
    out[r * 2 * hidden + c] = from_float<A>(a[i]);
    out[r * 2 * hidden + hidden + c] = from_float<A>(b[i]);
  }
}

}  // namespace psamd

using namespace psamd;

extern "C" {

const char* psamd_last_error(void) { return g_error.c_str(); }

int psamd_embed(void* stream, const int32_t* ids, const void* table, int table_dtype, float* out, int64_t tokens,
                int hidden, int vocab) {
  PSAMD_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (table_dtype == kBF16) {
    embed_kernel<bf16_t><<<dim3(tokens), dim3(256), 0, s>>>(ids, static_cast<const bf16_t*>(table), out, hidden, vocab);
  } else if (table_dtype == kF32) {
    embed_kernel<float><<<dim3(tokens), dim3(256), 0, s>>>(ids, static_cast<const float*>(table), out, hidden, vocab);
  } else {
    return fail("psamd_embed: table dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_embed");
}

int psamd_add_rmsnorm(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                      int64_t partial_stride, const int32_t* rows, const void* weight, int weight_dtype, float eps,
                      void* out, int act_dtype, int64_t out_rows, int hidden) {
  PSAMD_REQUIRE(out_rows >= 0 && hidden > 0, "bad sizes");
  PSAMD_REQUIRE(weight_dtype == kF32 || weight_dtype == kBF16, "weight dtype must be float32 or bfloat16");
  PSAMD_REQUIRE(delta == nullptr || delta_dtype == kF32 || delta_dtype == kBF16, "delta dtype");
  PSAMD_REQUIRE(delta == nullptr || (n_partials >= 1 && (n_partials == 1 || delta_dtype == kF32)),
                "partial sums must be float32");
  if (out_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  constexpr int kThreads = 256, kCache = 16;
  const dim3 grid(static_cast<unsigned>(out_rows)), block(kThreads);
#define PSAMD_NORM(A_, D_)                                                                                      \
  add_rmsnorm_kernel<A_, D_, kThreads, kCache><<<grid, block, 0, s>>>(                                          \
      residual, static_cast<const D_*>(delta), n_partials, partial_stride, rows, weight, weight_dtype, eps, \
      static_cast<A_*>(out), hidden)
  const bool delta_f32 = delta == nullptr || delta_dtype == kF32;
  if (act_dtype == kBF16 && hidden % 8 == 0 && hidden <= 8 * kThreads * 4) {
    bf16_t* o16 = static_cast<bf16_t*>(out);
#define PSAMD_NORM8(D_, IT_)                                                                                 \
  add_rmsnorm_vec8_kernel<D_, kThreads, IT_><<<grid, block, 0, s>>>(                                         \
      residual, static_cast<const D_*>(delta), n_partials, partial_stride, rows, weight, weight_dtype, eps, \
      o16, hidden)
    const int iters = static_cast<int>(ceil_div(hidden / 8, kThreads));
    if (delta_f32) {
      if (iters <= 1) PSAMD_NORM8(float, 1); else if (iters <= 2) PSAMD_NORM8(float, 2); else PSAMD_NORM8(float, 4);
    } else {
      if (iters <= 1) PSAMD_NORM8(bf16_t, 1); else if (iters <= 2) PSAMD_NORM8(bf16_t, 2); else PSAMD_NORM8(bf16_t, 4);
    }
#undef PSAMD_NORM8
    return check_launch("psamd_add_rmsnorm");
  }
  if (act_dtype == kBF16) {
    if (delta_f32) PSAMD_NORM(bf16_t, float); else PSAMD_NORM(bf16_t, bf16_t);
  } else if (act_dtype == kF32) {
    if (delta_f32) PSAMD_NORM(float, float); else PSAMD_NORM(float, bf16_t);
  } else {
    return fail("psamd_add_rmsnorm: activation dtype must be float32 or bfloat16");
  }
#undef PSAMD_NORM
  return check_launch("psamd_add_rmsnorm");
}

int psamd_swiglu(void* stream, const void* gate_up, void* out, int act_dtype, int64_t tokens, int inter, int gate) {
  PSAMD_REQUIRE(tokens >= 0 && inter > 0, "bad sizes");
  PSAMD_REQUIRE(gate >= 0 && gate <= 2, "the gate's activation is 0 (SiLU), 1 (ReLU) or 2 (GELU, tanh form)");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = tokens * inter;
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  if (act_dtype == kBF16 && inter % 8 == 0) {
    const int vblocks = static_cast<int>(std::min<int64_t>(ceil_div(n / 8, 256), 65536));
    swiglu_vec8_kernel<<<dim3(vblocks), dim3(256), 0, s>>>(static_cast<const bf16_t*>(gate_up),
                                                           static_cast<bf16_t*>(out), tokens, inter, gate);
  } else if (act_dtype == kBF16) {
    swiglu_kernel<bf16_t><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const bf16_t*>(gate_up),
                                                            static_cast<bf16_t*>(out), tokens, inter, gate);
  } else if (act_dtype == kF32) {
    swiglu_kernel<float><<<dim3(blocks), dim3(256), 0, s>>>(static_cast<const float*>(gate_up),
                                                           static_cast<float*>(out), tokens, inter, gate);
  } else {
    return fail("psamd_swiglu: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_swiglu");
}

int psamd_rope_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                         const int32_t* positions, const float* table, void* kv, const int32_t* write_slot) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv > 0, "bad sizes");
  PSAMD_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "head_dim must be even");
  PSAMD_REQUIRE(kv == nullptr || write_slot != nullptr, "a cache needs write slots");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float2* tab = reinterpret_cast<const float2*>(table);
  if (act_dtype == kBF16 && head_dim % 16 == 0 && static_cast<size_t>(16) * (hkv * head_dim + 8) * sizeof(bf16_t) <= 64 * 1024) {
    const size_t smem = static_cast<size_t>(16) * (hkv * head_dim + 8) * sizeof(bf16_t);
    // Enough blocks for every compute unit, each with at least a round of work for its threads.
    const int64_t groups = ceil_div(tokens, 16);
    const int64_t rot_rounds = ceil_div(static_cast<int64_t>(16) * (hq + hkv) * (head_dim / 16), 256);
    const unsigned split = static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>({rot_rounds, 16, ceil_div(1024, groups)})));
    rope_kv_append_vec_kernel<<<dim3(static_cast<unsigned>(groups), split), dim3(256), smem, s>>>(
        static_cast<bf16_t*>(qkv), static_cast<int>(tokens), hq, hkv, head_dim, positions, tab, static_cast<bf16_t*>(kv),
        write_slot);
  } else if (act_dtype == kBF16) {
    rope_kv_append_kernel<bf16_t><<<dim3(tokens), dim3(256), 0, s>>>(static_cast<bf16_t*>(qkv), hq, hkv, head_dim,
                                                                    positions, tab, static_cast<bf16_t*>(kv), write_slot);
  } else if (act_dtype == kF32) {
    rope_kv_append_kernel<float><<<dim3(tokens), dim3(256), 0, s>>>(static_cast<float*>(qkv), hq, hkv, head_dim,
                                                                   positions, tab, static_cast<float*>(kv), write_slot);
  } else {
    return fail("psamd_rope_kv_append: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_rope_kv_append");
}

int psamd_scaled_add_rmsnorm(void* stream, float* residual, float alpha, const void* delta, int delta_dtype,
                             int n_partials, int64_t partial_stride, const void* weight, int weight_dtype, float eps,
                             void* out, int act_dtype, int64_t rows, int hidden) {
  PSAMD_REQUIRE(rows >= 0 && hidden > 0, "bad sizes");
  PSAMD_REQUIRE(weight_dtype == kF32 || weight_dtype == kBF16, "weight dtype must be float32 or bfloat16");
  PSAMD_REQUIRE(delta == nullptr || delta_dtype == kF32 || delta_dtype == kBF16, "delta dtype");
  PSAMD_REQUIRE(delta == nullptr || (n_partials >= 1 && (n_partials == 1 || delta_dtype == kF32)),
                "partial sums must be float32");
  PSAMD_REQUIRE(out == nullptr || act_dtype == kF32 || act_dtype == kBF16, "activation dtype");
  if (rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  constexpr int kThreads = 256, kCache = 16;
  const dim3 grid(static_cast<unsigned>(rows)), block(kThreads);
#define PSAMD_POSTNORM(A_, D_)                                                                              \
  scaled_add_rmsnorm_kernel<A_, D_, kThreads, kCache><<<grid, block, 0, s>>>(                               \
      residual, alpha, static_cast<const D_*>(delta), n_partials, partial_stride, weight, weight_dtype, eps, \
      static_cast<A_*>(out), hidden)
  const bool delta_f32 = delta == nullptr || delta_dtype == kF32;
  const bool out_bf16 = out != nullptr && act_dtype == kBF16;
  if (hidden % 4 == 0 && hidden <= 4 * kThreads * 8 && (partial_stride % 4 == 0 || n_partials <= 1)) {
#define PSAMD_POSTNORM4(A_, D_, IT_)                                                                        \
  scaled_add_rmsnorm_vec4_kernel<A_, D_, kThreads, IT_><<<grid, block, 0, s>>>(                             \
      residual, alpha, static_cast<const D_*>(delta), n_partials, partial_stride, weight, weight_dtype, eps, \
      static_cast<A_*>(out), hidden)
#define PSAMD_POSTNORM4_IT(A_, D_)                                                 \
  do {                                                                             \
    if (hidden <= 4 * kThreads * 2) PSAMD_POSTNORM4(A_, D_, 2);                    \
    else if (hidden <= 4 * kThreads * 4) PSAMD_POSTNORM4(A_, D_, 4);               \
    else PSAMD_POSTNORM4(A_, D_, 8);                                               \
  } while (0)
    if (out_bf16) {
      if (delta_f32) PSAMD_POSTNORM4_IT(bf16_t, float); else PSAMD_POSTNORM4_IT(bf16_t, bf16_t);
    } else {
      if (delta_f32) PSAMD_POSTNORM4_IT(float, float); else PSAMD_POSTNORM4_IT(float, bf16_t);
    }
#undef PSAMD_POSTNORM4_IT
#undef PSAMD_POSTNORM4
    return check_launch("psamd_scaled_add_rmsnorm");
  }
  if (out_bf16) {
    if (delta_f32) PSAMD_POSTNORM(bf16_t, float); else PSAMD_POSTNORM(bf16_t, bf16_t);
  } else {
    if (delta_f32) PSAMD_POSTNORM(float, float); else PSAMD_POSTNORM(float, bf16_t);
  }
#undef PSAMD_POSTNORM
  return check_launch("psamd_scaled_add_rmsnorm");
}

int psamd_to_activation(void* stream, const float* in, void* out, int act_dtype, int64_t n) {
  PSAMD_REQUIRE(n >= 0, "bad size");
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  if (act_dtype == kBF16) {
    to_activation_kernel<bf16_t><<<dim3(blocks), dim3(256), 0, s>>>(in, static_cast<bf16_t*>(out), n);
  } else if (act_dtype == kF32) {
    to_activation_kernel<float><<<dim3(blocks), dim3(256), 0, s>>>(in, static_cast<float*>(out), n);
  } else {
    return fail("psamd_to_activation: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_to_activation");
}

int psamd_qk_prepare_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                               const int32_t* positions, const float* table, int norm_dim, float eps, const float* bias,
                               const float* q_weight, const float* k_weight, int v_from_k, void* kv,
                               const int32_t* write_slot, int q_weight_per_head) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv >= 0, "bad sizes");
  const int q_weight_stride = q_weight_per_head ? head_dim : 0;
  PSAMD_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 256, "head_dim must be even and at most 256");
  PSAMD_REQUIRE(norm_dim >= 0 && norm_dim <= head_dim, "norm_dim must be in [0, head_dim]");
  PSAMD_REQUIRE(kv == nullptr || (write_slot != nullptr && hkv > 0), "a cache needs write slots and kv heads");
  PSAMD_REQUIRE(tokens <= 2147483647LL, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float2* tab = reinterpret_cast<const float2*>(table);
  const int row_heads = hq + (v_from_k ? hkv : 2 * hkv);
  int group_lanes = 1;                                   // lanes per head: the power of two that holds d/2 pairs, up to a wave
  while (group_lanes < 64 && group_lanes < head_dim / 2) group_lanes *= 2;
  const int heads_per_block = 4 * (64 / group_lanes);
  PSAMD_REQUIRE(ceil_div(row_heads, heads_per_block) <= 65535, "too many heads for one launch");
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(ceil_div(row_heads, heads_per_block)));
  if (act_dtype == kBF16) {
    rope_norm_kv_append_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<bf16_t*>(qkv), hq, hkv, head_dim, positions,
                                                                 tab, norm_dim, eps, static_cast<bf16_t*>(kv), write_slot,
                                                                 group_lanes, bias, q_weight, k_weight, v_from_k, q_weight_stride);
  } else if (act_dtype == kF32) {
    rope_norm_kv_append_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<float*>(qkv), hq, hkv, head_dim, positions,
                                                                tab, norm_dim, eps, static_cast<float*>(kv), write_slot,
                                                                group_lanes, bias, q_weight, k_weight, v_from_k, q_weight_stride);
  } else {
    return fail("psamd_qk_prepare_kv_append: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_qk_prepare_kv_append");
}

int psamd_rope_norm_kv_append(void* stream, void* qkv, int act_dtype, int64_t tokens, int hq, int hkv, int head_dim,
                              const int32_t* positions, const float* table, int norm_dim, float eps, void* kv,
                              const int32_t* write_slot) {
  return psamd_qk_prepare_kv_append(stream, qkv, act_dtype, tokens, hq, hkv, head_dim, positions, table, norm_dim, eps,
                                    nullptr, nullptr, nullptr, 0, kv, write_slot, 0);
}

// residual[r] += delta[r] (delta as for psamd_add_rmsnorm: one tensor in delta_dtype or float32 slices).
int psamd_residual_add(void* stream, float* residual, const void* delta, int delta_dtype, int n_partials,
                       int64_t partial_stride, int64_t rows, int hidden) {
  PSAMD_REQUIRE(rows >= 0 && hidden > 0 && n_partials >= 1 && delta != nullptr, "bad sizes");
  PSAMD_REQUIRE(n_partials == 1 || delta_dtype == kF32, "partial sums are float32");
  if (rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = rows * hidden;
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  if (delta_dtype == kBF16) {
    residual_add_kernel<bf16_t><<<dim3(blocks), dim3(256), 0, s>>>(residual, static_cast<const bf16_t*>(delta), n_partials,
                                                                  partial_stride, n);
  } else if (delta_dtype == kF32) {
    residual_add_kernel<float><<<dim3(blocks), dim3(256), 0, s>>>(residual, static_cast<const float*>(delta), n_partials,
                                                                 partial_stride, n);
  } else {
    return fail("psamd_residual_add: delta dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_residual_add");
}

// x[r, c] = x[r, c] * factor + (row != NULL ? row[c] : 0), in float32.
int psamd_stream_affine(void* stream, float* x, int64_t rows, int hidden, float factor, const float* row) {
  PSAMD_REQUIRE(rows >= 0 && hidden > 0, "bad sizes");
  if (rows == 0) return 0;
  const int64_t n = rows * hidden;
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  stream_affine_kernel<<<dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, n, hidden, factor, row);
  return check_launch("psamd_stream_affine");
}

// out[r] = [a[r], b[r]] in act_dtype: two float32 streams side by side as one product's input.
int psamd_concat_to_activation(void* stream, const float* a, const float* b, void* out, int act_dtype, int64_t rows,
                               int hidden) {
  PSAMD_REQUIRE(rows >= 0 && hidden > 0, "bad sizes");
  if (rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = rows * hidden;
  const int blocks = static_cast<int>(std::min<int64_t>(ceil_div(n, 256), 65536));
  if (act_dtype == kBF16) {
    concat_to_activation_kernel<bf16_t><<<dim3(blocks), dim3(256), 0, s>>>(a, b, static_cast<bf16_t*>(out), n, hidden);
  } else if (act_dtype == kF32) {
    concat_to_activation_kernel<float><<<dim3(blocks), dim3(256), 0, s>>>(a, b, static_cast<float*>(out), n, hidden);
  } else {
    return fail("psamd_concat_to_activation: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_concat_to_activation");
}

}  // extern "C"
