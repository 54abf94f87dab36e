// Delta-rule mixers: a matrix state per head that is decayed, has one direction partly removed and
// one outer product written per token, and is read with a query.
//
// The recurrence all forms share, per head, with S [dim, vdim] in float:
//     S' = diag(d) S                       d: a vector per key channel, or one number per head, or both
//     S  = S' + (ps p) (c^T S*) + k (xs x)^T        S* = S (the state before the decay) or S'
//     o  = S^T r
// * gated delta rule: d = g (a number), p = c = k (a unit vector), ps = -b, xs = b, S* = S':
//   S <- g S; S <- S + k (b (v - S^T k))^T; the output reads the state after the write.
// * generalized delta rule: d = w (a vector), c = k / |k|, p = -(a * c), ps = xs = 1, S* = S:
//   S <- diag(w) S - (a * c)(c^T S) + k v^T.
// Every column of S (one value channel) goes its own way, so a column is dealt out to 16 lanes and a
// workgroup holds 16 columns of one (item, head) in registers while it walks the item's tokens; the
// vectors of a run of tokens are staged in LDS once for all 16 columns. Everything is float whatever
// the activation type: decays, strengths, unit vectors, sums, the state. A step continues from
// state[slot] and leaves the new state there; the runner hands a request that starts at position 0
// a zeroed slot. The state of a head is stored [vdim][dim], so a column is contiguous.
//
// In front of the recurrence: a short causal convolution per channel (continued across steps from the
// inputs the state saved) with SiLU, and the kernels that turn the projections into the recurrence's
// operands. Behind it: an RMS norm per head times a weight times an activation of a gate.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kConvMaxTaps = 16;
constexpr int kLPC = 16;      // lanes per column of the state
constexpr int kCols = 16;     // columns per workgroup

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ------------------------------------------------------------------ short convolution

// grid (tokens + items, ceil(channels / 256)). A token that lies taps - 1 or more behind its item's
// first token needs nothing but the step's own rows: one thread per (token, channel). The first
// taps - 1 tokens of an item read the inputs the state saved, and the state's saved inputs are
// replaced by the item's last ones: both are the work of one thread per (item, channel), so that
// nobody reads a saved input another thread has already replaced.
template <typename A>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const A* __restrict__ in, int64_t in_row, const float* __restrict__ w, float* __restrict__ out, int64_t out_row,
    float* __restrict__ state, int64_t state_row, const int32_t* __restrict__ tok_item,
    const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots, int tokens, int channels, int taps, int act) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int keep = taps - 1;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  if (static_cast<int>(blockIdx.x) < tokens) {
    const int64_t t = blockIdx.x;
    const int64_t s0 = item_start[tok_item[t]];
    if (t - s0 < keep) return;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) acc = fmaf(wc[j], to_float<A>(in[(t - keep + j) * in_row + c]), acc);
    out[t * out_row + c] = act ? acc * sigmoidf_(acc) : acc;
    return;
  }
  const int item = static_cast<int>(blockIdx.x) - tokens;
  const int64_t s0 = item_start[item];
  const int n = static_cast<int>(item_start[item + 1] - s0);
  float* saved = state + static_cast<int64_t>(slots[item]) * state_row + c;      // saved[j * channels]: oldest first
  const int first = min(n, keep);
  for (int li = 0; li < first; ++li) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = li - keep + j;
      const float v = src >= 0 ? to_float<A>(in[(s0 + src) * in_row + c]) : saved[static_cast<int64_t>(keep + src) * channels];
      acc = fmaf(wc[j], v, acc);
    }
    out[(s0 + li) * out_row + c] = act ? acc * sigmoidf_(acc) : acc;
  }
  // The new saved inputs, oldest first: entry j is the input n - keep + j of the item, or a saved one
  // further back. Ascending j reads saved entries at or behind the one it writes.
  for (int j = 0; j < keep; ++j) {
    const int src = n - keep + j;
    saved[static_cast<int64_t>(j) * channels] =
        src >= 0 ? to_float<A>(in[(s0 + src) * in_row + c]) : saved[static_cast<int64_t>(keep + src) * channels];
  }
}

// ------------------------------------------------------------------ operands of the gated delta rule

// grid (tokens), 256 threads. u row = [q: groups x dim | k: groups x dim | values]: every q and k
// vector is divided by sqrt(sum of squares + unit_eps) in place, q also times q_scale. gates row =
// [strength logits: heads | decay inputs: heads] -> coef row = [g | -b | b], heads each, with
// b = sigmoid(.), g = exp(-exp(a_log[h]) softplus(. + dt_bias[h])).
__global__ __launch_bounds__(256) void gated_delta_prepare_kernel(
    float* __restrict__ u, int64_t u_row, int groups, int dim, const float* __restrict__ gates,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ coef, int heads, float q_scale,
    float unit_eps) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  for (int v = wave; v < 2 * groups; v += 4) {          // q vectors, then k vectors
    float* p = u + t * u_row + static_cast<int64_t>(v) * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += kWave) ss = fmaf(p[i], p[i], ss);
    ss = wave_sum(ss);
    const float f = (v < groups ? q_scale : 1.f) / sqrtf(ss + unit_eps);
    for (int i = lane; i < dim; i += kWave) p[i] *= f;
  }
  for (int h = threadIdx.x; h < heads; h += blockDim.x) {
    const float b = sigmoidf_(gates[t * 2 * heads + h]);
    const float g = expf(-expf(a_log[h]) * softplusf_(gates[t * 2 * heads + heads + h] + dt_bias[h]));
    float* c = coef + t * 3 * heads;
    c[h] = g;
    c[heads + h] = -b;
    c[2 * heads + h] = b;
  }
}

// ------------------------------------------------------------------ operands of the generalized delta rule

// grid (tokens, heads), 256 threads over the head's channels. rows (activation type) hold r, k, v,
// the removal rate's logits (heads x dim each, at their columns) and the low-rank map's inner
// values (rank, at l_col). ops row = [r | k | v | w | p | c], heads x dim each, float:
//   w = exp(-decay_floor * sigmoid(sum_j w2[hc, j] tanh(l[j]) + w0[hc])), c = k / sqrt(sum k^2 + unit_eps),
//   p = -sigmoid(a + a_bias[hc]) * c.
template <typename A>
__global__ __launch_bounds__(256) void general_delta_prepare_kernel(
    const A* __restrict__ rows, int64_t in_row, int r_col, int k_col, int v_col, int a_col, int l_col,
    const float* __restrict__ a_bias, const float* __restrict__ w2, const float* __restrict__ w0, float* __restrict__ ops,
    int heads, int dim, int rank, float decay_floor, float unit_eps) {
  extern __shared__ float prep_smem[];                 // tanh(l)[rank], then 4 floats for the sum
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const A* row = rows + t * in_row;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) prep_smem[j] = tanhf(to_float<A>(row[l_col + j]));
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const float k = to_float<A>(row[k_col + h * dim + i]);
    ss = fmaf(k, k, ss);
  }
  ss = block_sum(ss, prep_smem + rank, 4);             // its barriers also publish the tanh values
  const float inv = 1.f / sqrtf(ss + unit_eps);
  const int64_t hd = static_cast<int64_t>(heads) * dim;
  float* o = ops + t * 6 * hd + static_cast<int64_t>(h) * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) {
    const int64_t hc = static_cast<int64_t>(h) * dim + i;
    const float* w2r = w2 + hc * rank;
    float low = w0[hc];
    for (int j = 0; j < rank; ++j) low = fmaf(w2r[j], prep_smem[j], low);
    const float k = to_float<A>(row[k_col + hc]);
    const float c = k * inv;
    o[i] = to_float<A>(row[r_col + hc]);
    o[hd + i] = k;
    o[2 * hd + i] = to_float<A>(row[v_col + hc]);
    o[3 * hd + i] = expf(-decay_floor * sigmoidf_(low));
    o[4 * hd + i] = -sigmoidf_(to_float<A>(row[a_col + hc]) + a_bias[hc]) * c;
    o[5 * hd + i] = c;
  }
}

// ------------------------------------------------------------------ the recurrence

// grid (items, heads, ceil(vdim / 16)), 256 threads: column col = threadIdx.x / 16 of the block's 16,
// lane l of its 16 holds the E entries l * E .. l * E + E - 1 of the column (dim <= 16 E). The vectors
// of `tt` tokens at a time pass through LDS.
template <int E>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const float* __restrict__ kvec, const float* __restrict__ cvec, const float* __restrict__ pvec,
    const float* __restrict__ rvec, int64_t key_row, int heads_per_group, const float* __restrict__ dvec, int64_t dvec_row,
    const float* __restrict__ dscal, const float* __restrict__ pscal, const float* __restrict__ xscal, int64_t scal_row,
    const float* __restrict__ x, int64_t x_row, float* __restrict__ out, int64_t out_row, float* __restrict__ state,
    int64_t state_row, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots, int dim, int vdim,
    int reads_decayed, int tt) {
  constexpr int DP = E * kLPC;                          // the column's length, padded
  extern __shared__ __align__(16) float scan_smem[];   // [tt][5][DP] k, c, p, r, d; [tt][4] d, ps, xs; [tt][kCols] x
  float* vec = scan_smem;
  float* sca = vec + static_cast<int64_t>(tt) * 5 * DP;
  float* xs_ = sca + tt * 4;
  const int item = blockIdx.x, h = blockIdx.y, g = h / heads_per_group;
  const int col = threadIdx.x / kLPC, l = threadIdx.x % kLPC;
  const int j0 = blockIdx.z * kCols, j = j0 + col;
  const int64_t s0 = item_start[item], s1 = item_start[item + 1];
  float* st = state + static_cast<int64_t>(slots[item]) * state_row + (static_cast<int64_t>(h) * vdim + j) * dim + l * E;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = (j < vdim && l * E + e < dim) ? st[e] : 0.f;
  for (int64_t t0 = s0; t0 < s1; t0 += tt) {
    const int n = static_cast<int>(min(static_cast<int64_t>(tt), s1 - t0));
    __syncthreads();                                    // everybody is done with the run before
    for (int idx = threadIdx.x; idx < n * DP; idx += 256) {
      const int tk = idx / DP, i = idx % DP;
      const int64_t at = (t0 + tk) * key_row + static_cast<int64_t>(g) * dim + i;
      const bool in = i < dim;
      float* v = vec + (static_cast<int64_t>(tk) * 5) * DP + i;
      v[0] = in ? kvec[at] : 0.f;
      v[DP] = in ? cvec[at] : 0.f;
      v[2 * DP] = in ? pvec[at] : 0.f;
      v[3 * DP] = in ? rvec[at] : 0.f;
      v[4 * DP] = (in && dvec != nullptr) ? dvec[(t0 + tk) * dvec_row + static_cast<int64_t>(h) * dim + i] : 1.f;
    }
    for (int idx = threadIdx.x; idx < n; idx += 256) {
      const int64_t at = (t0 + idx) * scal_row + h;
      sca[idx * 4] = dscal != nullptr ? dscal[at] : 1.f;
      sca[idx * 4 + 1] = pscal != nullptr ? pscal[at] : 1.f;
      sca[idx * 4 + 2] = xscal != nullptr ? xscal[at] : 1.f;
    }
    for (int idx = threadIdx.x; idx < n * kCols; idx += 256) {
      const int tk = idx / kCols, cc = idx % kCols;
      xs_[idx] = j0 + cc < vdim ? x[(t0 + tk) * x_row + static_cast<int64_t>(h) * vdim + j0 + cc] : 0.f;
    }
    __syncthreads();
    for (int tk = 0; tk < n; ++tk) {
      const float* v = vec + (static_cast<int64_t>(tk) * 5) * DP + l * E;
      const float ds = sca[tk * 4], ps = sca[tk * 4 + 1], xw = sca[tk * 4 + 2] * xs_[tk * kCols + col];
      float dec[E];
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        dec[e] = v[4 * DP + e] * ds * s[e];
        dot = fmaf(v[DP + e], reads_decayed ? dec[e] : s[e], dot);
      }
#pragma unroll
      for (int o = kLPC / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o, kWave);
      const float take = ps * dot;
      float read = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        s[e] = fmaf(v[e], xw, fmaf(v[2 * DP + e], take, dec[e]));
        read = fmaf(v[3 * DP + e], s[e], read);
      }
#pragma unroll
      for (int o = kLPC / 2; o > 0; o >>= 1) read += __shfl_xor(read, o, kWave);
      if (l == 0 && j < vdim) out[(t0 + tk) * out_row + static_cast<int64_t>(h) * vdim + j] = read;
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e)
    if (j < vdim && l * E + e < dim) st[e] = s[e];
}

// ------------------------------------------------------------------ norm per head, weight, gate

// One wave per (token, head): out = o / sqrt(mean(o^2) + eps) * weight * act(gate), act 0 = SiLU,
// 1 = sigmoid. weight is [vdim] shared by the heads, or [heads * vdim] (weight_head = vdim).
template <typename A>
__global__ __launch_bounds__(256) void heads_norm_gate_kernel(const float* __restrict__ o, int64_t pairs, int heads, int vdim,
                                                              const float* __restrict__ weight, int weight_head, float eps,
                                                              const A* __restrict__ gate, int64_t gate_row, int gate_act,
                                                              A* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t pair = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int64_t t = pair / heads;
  const int h = static_cast<int>(pair - t * heads);
  const float* src = o + pair * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += kWave) ss = fmaf(src[i], src[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(vdim) + eps);
  const A* gp = gate + t * gate_row + static_cast<int64_t>(h) * vdim;
  const float* wp = weight + static_cast<int64_t>(h) * weight_head;
  for (int i = lane; i < vdim; i += kWave) {
    const float z = to_float<A>(gp[i]);
    const float sg = sigmoidf_(z);
    out[pair * vdim + i] = from_float<A>(src[i] * inv * wp[i] * (gate_act == 0 ? z * sg : sg));
  }
}

template <int E>
static int launch_delta_scan(hipStream_t s, dim3 grid, size_t smem, const float* kvec, const float* cvec, const float* pvec,
                             const float* rvec, int64_t key_row, int heads_per_group, const float* dvec, int64_t dvec_row,
                             const float* dscal, const float* pscal, const float* xscal, int64_t scal_row, const float* x,
                             int64_t x_row, float* out, int64_t out_row, float* state, int64_t state_row,
                             const int32_t* item_start, const int32_t* slots, int dim, int vdim, int reads_decayed, int tt) {
  delta_scan_kernel<E><<<grid, dim3(256), smem, s>>>(kvec, cvec, pvec, rvec, key_row, heads_per_group, dvec, dvec_row, dscal,
                                                     pscal, xscal, scal_row, x, x_row, out, out_row, state, state_row,
                                                     item_start, slots, dim, vdim, reads_decayed, tt);
  return check_launch("psamd_delta_scan");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_short_conv(void* stream, const void* in, int act_dtype, int64_t in_row, const float* taps_w, float* out,
                     int64_t out_row, float* state, int64_t state_row, const int32_t* tok_item, const int32_t* item_start,
                     const int32_t* slots, int64_t tokens, int items, int channels, int taps, int act) {
  PSAMD_REQUIRE(tokens >= 0 && items >= 0 && channels > 0 && taps >= 1 && taps <= kConvMaxTaps, "bad sizes (at most 16 taps)");
  PSAMD_REQUIRE(in_row >= channels && out_row >= channels && state_row >= static_cast<int64_t>(taps - 1) * channels,
                "rows too short");
  PSAMD_REQUIRE(tokens + items <= 2147483647LL && ceil_div(channels, 256) <= 65535, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens + items), static_cast<unsigned>(ceil_div(channels, 256)));
  if (act_dtype == kBF16) {
    short_conv_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(in), in_row, taps_w, out, out_row, state,
                                                        state_row, tok_item, item_start, slots, static_cast<int>(tokens),
                                                        channels, taps, act);
  } else if (act_dtype == kF32) {
    short_conv_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(in), in_row, taps_w, out, out_row, state,
                                                       state_row, tok_item, item_start, slots, static_cast<int>(tokens),
                                                       channels, taps, act);
  } else {
    return fail("psamd_short_conv: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_short_conv");
}

int psamd_gated_delta_prepare(void* stream, float* u, int64_t u_row, int groups, int dim, const float* gates,
                              const float* a_log, const float* dt_bias, float* coef, int64_t tokens, int heads,
                              float q_scale, float unit_eps) {
  PSAMD_REQUIRE(tokens >= 0 && groups > 0 && dim > 0 && heads > 0, "bad sizes");
  PSAMD_REQUIRE(u_row >= 2LL * groups * dim && tokens <= 2147483647LL, "rows too short or too many tokens");
  if (tokens == 0) return 0;
  gated_delta_prepare_kernel<<<dim3(static_cast<unsigned>(tokens)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
      u, u_row, groups, dim, gates, a_log, dt_bias, coef, heads, q_scale, unit_eps);
  return check_launch("psamd_gated_delta_prepare");
}

int psamd_general_delta_prepare(void* stream, const void* rows, int act_dtype, int64_t in_row, int r_col, int k_col,
                                int v_col, int a_col, int l_col, const float* a_bias, const float* w2, const float* w0,
                                float* ops, int64_t tokens, int heads, int dim, int rank, float decay_floor, float unit_eps) {
  PSAMD_REQUIRE(tokens >= 0 && heads > 0 && dim > 0 && rank > 0, "bad sizes");
  PSAMD_REQUIRE(tokens <= 2147483647LL && heads <= 65535 && rank <= 8192, "too large for one launch");
  const int64_t hd = static_cast<int64_t>(heads) * dim;
  PSAMD_REQUIRE(std::max(std::max(r_col, k_col), std::max(v_col, a_col)) + hd <= in_row && l_col + rank <= in_row &&
                    std::min(std::min(std::min(r_col, k_col), std::min(v_col, a_col)), l_col) >= 0,
                "columns outside the rows");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(heads));
  const size_t smem = sizeof(float) * (static_cast<size_t>(rank) + 4);
  if (act_dtype == kBF16) {
    general_delta_prepare_kernel<bf16_t><<<grid, dim3(256), smem, s>>>(static_cast<const bf16_t*>(rows), in_row, r_col, k_col,
                                                                      v_col, a_col, l_col, a_bias, w2, w0, ops, heads, dim,
                                                                      rank, decay_floor, unit_eps);
  } else if (act_dtype == kF32) {
    general_delta_prepare_kernel<float><<<grid, dim3(256), smem, s>>>(static_cast<const float*>(rows), in_row, r_col, k_col,
                                                                     v_col, a_col, l_col, a_bias, w2, w0, ops, heads, dim, rank,
                                                                     decay_floor, unit_eps);
  } else {
    return fail("psamd_general_delta_prepare: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_general_delta_prepare");
}

int psamd_delta_scan(void* stream, const float* kvec, const float* cvec, const float* pvec, const float* rvec, int64_t key_row,
                     int key_groups, const float* dvec, int64_t dvec_row, const float* dscal, const float* pscal,
                     const float* xscal, int64_t scal_row, const float* x, int64_t x_row, float* out, int64_t out_row,
                     float* state, int64_t state_row, const int32_t* item_start, const int32_t* slots, int items, int heads,
                     int dim, int vdim, int reads_decayed) {
  PSAMD_REQUIRE(items >= 0 && heads > 0 && key_groups > 0 && heads % key_groups == 0 && dim > 0 && vdim > 0, "bad sizes");
  PSAMD_REQUIRE(dim <= 16 * kLPC, "key size at most 256");
  PSAMD_REQUIRE(state_row >= static_cast<int64_t>(heads) * dim * vdim, "state rows too short");
  PSAMD_REQUIRE(heads <= 65535 && ceil_div(vdim, kCols) <= 65535, "too large for one launch");
  PSAMD_REQUIRE(kvec && cvec && pvec && rvec && x && out && state, "missing operands");
  if (items == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int e = 1;
  while (e * kLPC < dim) e *= 2;
  const int dp = e * kLPC;
  const size_t per_token = sizeof(float) * (5 * static_cast<size_t>(dp) + 4 + kCols);
  const int tt = static_cast<int>(std::max<size_t>(1, std::min<size_t>(16, (48 * 1024) / per_token)));
  const size_t smem = per_token * tt;
  const dim3 grid(static_cast<unsigned>(items), static_cast<unsigned>(heads), static_cast<unsigned>(ceil_div(vdim, kCols)));
  const int hpg = heads / key_groups;
#define PSAMD_SCAN(E)                                                                                                  \
  return launch_delta_scan<E>(s, grid, smem, kvec, cvec, pvec, rvec, key_row, hpg, dvec, dvec_row, dscal, pscal, xscal,  \
                              scal_row, x, x_row, out, out_row, state, state_row, item_start, slots, dim, vdim,        \
                              reads_decayed, tt)
  switch (e) {
    case 1: PSAMD_SCAN(1);
    case 2: PSAMD_SCAN(2);
    case 4: PSAMD_SCAN(4);
    case 8: PSAMD_SCAN(8);
    default: PSAMD_SCAN(16);
  }
#undef PSAMD_SCAN
}

int psamd_heads_norm_gate(void* stream, const float* o, int64_t tokens, int heads, int vdim, const float* weight,
                          int weight_per_head, float eps, const void* gate, int act_dtype, int64_t gate_row, int gate_act,
                          void* out) {
  PSAMD_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0 && gate_row >= static_cast<int64_t>(heads) * vdim, "bad sizes");
  PSAMD_REQUIRE(gate_act == 0 || gate_act == 1, "the gate's activation is SiLU (0) or sigmoid (1)");
  const int64_t pairs = tokens * heads;
  PSAMD_REQUIRE(ceil_div(pairs, 4) <= 2147483647LL, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(ceil_div(pairs, 4)));
  const int wh = weight_per_head ? vdim : 0;
  if (act_dtype == kBF16) {
    heads_norm_gate_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(o, pairs, heads, vdim, weight, wh, eps,
                                                             static_cast<const bf16_t*>(gate), gate_row, gate_act,
                                                             static_cast<bf16_t*>(out));
  } else if (act_dtype == kF32) {
    heads_norm_gate_kernel<float><<<grid, dim3(256), 0, s>>>(o, pairs, heads, vdim, weight, wh, eps,
                                                            static_cast<const float*>(gate), gate_row, gate_act,
                                                            static_cast<float*>(out));
  } else {
    return fail("psamd_heads_norm_gate: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_heads_norm_gate");
}

}  // extern "C"
