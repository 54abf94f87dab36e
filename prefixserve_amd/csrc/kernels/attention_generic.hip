// Causal grouped-query attention over the paged cache, the straightforward way: one wave
// per (new token, query head), float arithmetic throughout, any head size up to 512, any number
// of heads and groups, optional sliding window, an optional
// learned sink per head (a term exp(sink) in the softmax's denominator that has no key and no
// value) and an optional bias on the scaled score that depends on the head and on how far back
// the key lies (a table per head, its last entry standing for every larger distance).
// It is the attention of the exact 32-bit path and the fallback for shapes the
// matrix-core kernels do not take.
//
// Page layout (per layer): [num_blocks][2][kv_heads][16 * D]; half 0 = keys [16][D],
// half 1 = values transposed [D][16].

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kMaxHead = 512;          // head sizes up to here: kMaxHead / 64 output dimensions per lane

template <typename A>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const A* __restrict__ qkv, int q_stride, A* __restrict__ out, const A* __restrict__ kv,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_item,
    const int32_t* __restrict__ table_off, const int32_t* __restrict__ block_ids,
    int hq, int hkv, int d, float scale, int window, const float* __restrict__ sink,
    const float* __restrict__ dist_bias, int n_dist) {
  __shared__ float q_s[kMaxHead];
  __shared__ float p_s[kWave];
  __shared__ int32_t base_s[kWave];   // element offset of (page, kv head) for each key of the chunk
  __shared__ int32_t off_s[kWave];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (hq / hkv);
  const int pos = positions[t];
  const int item = tok_item[t];
  const int32_t* table = block_ids + table_off[item];
  const int k_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int64_t page_elems = 2LL * hkv * kPage * d;
  const int64_t half_elems = static_cast<int64_t>(hkv) * kPage * d;

  const A* q = qkv + t * q_stride + h * d;
  for (int i = lane; i < d; i += kWave) q_s[i] = to_float<A>(q[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxHead / kWave] = {};      // dims lane, lane+64, lane+128, ...
  for (int c0 = k_lo; c0 <= pos; c0 += kWave) {
    const int j = c0 + lane;
    float s = -INFINITY;
    if (j <= pos) {
      const int64_t page = table[j / kPage];
      const int off = j % kPage;
      const int64_t base = page * page_elems + static_cast<int64_t>(kvh) * kPage * d;
      const A* kr = kv + base + static_cast<int64_t>(off) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float<A>(kr[i]), dot);
      s = dot * scale;
      if (dist_bias != nullptr) s += dist_bias[static_cast<int64_t>(h) * n_dist + min(pos - j, n_dist - 1)];
      base_s[lane] = static_cast<int32_t>(page);
      off_s[lane] = off;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = j <= pos ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);   // m = -inf on the first chunk gives 0
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    __syncthreads();
    const int cnt = min(kWave, pos - c0 + 1);
#pragma unroll
    for (int dd = 0; dd < kMaxHead / kWave; ++dd) {
      const int i = lane + dd * kWave;
      if (i < d) {
        float a = acc[dd] * alpha;
        for (int jj = 0; jj < cnt; ++jj) {
          const int64_t vb = static_cast<int64_t>(base_s[jj]) * page_elems + half_elems +
                             (static_cast<int64_t>(kvh) * d + i) * kPage + off_s[jj];
          a = fmaf(p_s[jj], to_float<A>(kv[vb]), a);
        }
        acc[dd] = a;
      }
    }
    __syncthreads();
  }
  if (sink != nullptr) l += expf(sink[h] - m);     // the query's own key is always seen: m is finite
  const float inv = 1.f / l;
  A* o = out + t * (static_cast<int64_t>(hq) * d) + h * d;
#pragma unroll
  for (int dd = 0; dd < kMaxHead / kWave; ++dd) {
    const int i = lane + dd * kWave;
    if (i < d) o[i] = from_float<A>(acc[dd] * inv);
  }
}

// The same wave per (new token, query head) for a sliding window with more to see than the window:
// the sequence's first `keep_first` positions stay visible at their true places, and with pooled
// blocks (pool != NULL) the query at position i also sees one mean key and value per block of
// `block` tokens that lies wholly in front of its window (block b once b * block + block - 1 <= i -
// window), read from pages of their own. All of them share one softmax. `gate` (float [tokens, hq]
// or NULL): the head's output times sigmoid(gate[t, h]).
// The visible keys are numbered 0 .. n - 1 in three runs: kept first positions in front of the
// window, the window's tokens, the pooled blocks; a lane takes one number per round of 64.
template <typename A>
__global__ __launch_bounds__(64) void attention_masked_kernel(
    const A* __restrict__ qkv, int q_stride, A* __restrict__ out, const A* __restrict__ kv,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ tok_item,
    const int32_t* __restrict__ table_off, const int32_t* __restrict__ block_ids,
    int hq, int hkv, int d, float scale, int window, int keep_first, const A* __restrict__ pool,
    const int32_t* __restrict__ pool_table_off, const int32_t* __restrict__ pool_block_ids, int block,
    const float* __restrict__ gate) {
  __shared__ float q_s[kMaxHead];
  __shared__ float p_s[kWave];
  __shared__ int64_t key_s[kWave];     // element offset of the key's row
  __shared__ int64_t val_s[kWave];     // element offset of the value's first dimension
  __shared__ int src_s[kWave];         // 0: token pages, 1: pool pages
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (hq / hkv);
  const int pos = positions[t];
  const int item = tok_item[t];
  const int32_t* table = block_ids + table_off[item];
  const int32_t* ptable = pool != nullptr ? pool_block_ids + pool_table_off[item] : nullptr;
  const int k_lo = max(0, pos - window + 1);
  const int n_first = min(keep_first, k_lo);
  const int n_win = pos - k_lo + 1;
  const int n_pool = pool != nullptr ? max(0, (pos - window + 1) / block) : 0;
  const int n_all = n_first + n_win + n_pool;
  const int64_t page_elems = 2LL * hkv * kPage * d;
  const int64_t half_elems = static_cast<int64_t>(hkv) * kPage * d;

  const A* q = qkv + t * q_stride + h * d;
  for (int i = lane; i < d; i += kWave) q_s[i] = to_float<A>(q[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxHead / kWave] = {};
  for (int c0 = 0; c0 < n_all; c0 += kWave) {
    const int v = c0 + lane;
    float s = -INFINITY;
    if (v < n_all) {
      const bool pooled = v >= n_first + n_win;
      const int j = v < n_first ? v : pooled ? v - n_first - n_win : k_lo + (v - n_first);
      const int64_t page = pooled ? ptable[j / kPage] : table[j / kPage];
      const int off = j % kPage;
      const int64_t base = page * page_elems + static_cast<int64_t>(kvh) * kPage * d;
      const A* kr = (pooled ? pool : kv) + base + static_cast<int64_t>(off) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float<A>(kr[i]), dot);
      s = dot * scale;
      key_s[lane] = base;
      val_s[lane] = base + half_elems + off;
      src_s[lane] = pooled ? 1 : 0;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = v < n_all ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    __syncthreads();
    const int cnt = min(kWave, n_all - c0);
#pragma unroll
    for (int dd = 0; dd < kMaxHead / kWave; ++dd) {
      const int i = lane + dd * kWave;
      if (i < d) {
        float a = acc[dd] * alpha;
        for (int jj = 0; jj < cnt; ++jj) {
          const A* vp = (src_s[jj] ? pool : kv) + val_s[jj] + static_cast<int64_t>(i) * kPage;
          a = fmaf(p_s[jj], to_float<A>(*vp), a);
        }
        acc[dd] = a;
      }
    }
    __syncthreads();
  }
  float inv = 1.f / l;
  if (gate != nullptr) inv *= 1.f / (1.f + expf(-gate[t * hq + h]));
  A* o = out + t * (static_cast<int64_t>(hq) * d) + h * d;
#pragma unroll
  for (int dd = 0; dd < kMaxHead / kWave; ++dd) {
    const int i = lane + dd * kWave;
    if (i < d) o[i] = from_float<A>(acc[dd] * inv);
  }
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_attention_generic(void* stream, const void* qkv, int q_stride, void* out, const void* kv,
                                       int act_dtype, int64_t tokens, const int32_t* positions,
                                       const int32_t* tok_item, const int32_t* table_off, const int32_t* block_ids,
                                       int hq, int hkv, int head_dim, float scale, int window, const float* sink,
                                       const float* dist_bias, int n_dist) {
  PSAMD_REQUIRE(dist_bias == nullptr || n_dist >= 1, "a distance bias needs at least one entry per head");
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv > 0 && hq % hkv == 0, "bad head counts");
  PSAMD_REQUIRE(head_dim > 0 && head_dim <= kMaxHead, "head_dim must be in [1, 512]");
  PSAMD_REQUIRE(hq <= 65535, "too many heads for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(hq));
  if (act_dtype == kBF16) {
    attention_generic_kernel<bf16_t><<<grid, dim3(64), 0, s>>>(
        static_cast<const bf16_t*>(qkv), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(kv),
        positions, tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window, sink, dist_bias, n_dist);
  } else if (act_dtype == kF32) {
    attention_generic_kernel<float><<<grid, dim3(64), 0, s>>>(
        static_cast<const float*>(qkv), q_stride, static_cast<float*>(out), static_cast<const float*>(kv),
        positions, tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window, sink, dist_bias, n_dist);
  } else {
    return fail("psamd_attention_generic: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_attention_generic");
}

extern "C" int psamd_attention_masked(void* stream, const void* qkv, int q_stride, void* out, const void* kv, int act_dtype,
                                      int64_t tokens, const int32_t* positions, const int32_t* tok_item,
                                      const int32_t* table_off, const int32_t* block_ids, int hq, int hkv, int head_dim,
                                      float scale, int window, int keep_first, const void* pool,
                                      const int32_t* pool_table_off, const int32_t* pool_block_ids, int block,
                                      const float* gate) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && hkv > 0 && hq % hkv == 0, "bad head counts");
  PSAMD_REQUIRE(head_dim > 0 && head_dim <= kMaxHead, "head_dim must be in [1, 512]");
  PSAMD_REQUIRE(hq <= 65535, "too many heads for one launch");
  PSAMD_REQUIRE(window >= 1 && keep_first >= 0, "kept first positions and pooled blocks belong to a window");
  PSAMD_REQUIRE(pool == nullptr || (block >= 1 && pool_table_off != nullptr && pool_block_ids != nullptr),
                "pooled blocks need their size and their pages' tables");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(hq));
  if (act_dtype == kBF16) {
    attention_masked_kernel<bf16_t><<<grid, dim3(64), 0, s>>>(
        static_cast<const bf16_t*>(qkv), q_stride, static_cast<bf16_t*>(out), static_cast<const bf16_t*>(kv), positions,
        tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window, keep_first, static_cast<const bf16_t*>(pool),
        pool_table_off, pool_block_ids, block, gate);
  } else if (act_dtype == kF32) {
    attention_masked_kernel<float><<<grid, dim3(64), 0, s>>>(
        static_cast<const float*>(qkv), q_stride, static_cast<float*>(out), static_cast<const float*>(kv), positions,
        tok_item, table_off, block_ids, hq, hkv, head_dim, scale, window, keep_first, static_cast<const float*>(pool),
        pool_table_off, pool_block_ids, block, gate);
  } else {
    return fail("psamd_attention_masked: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_attention_masked");
}
