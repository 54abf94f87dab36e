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
// Tokens whose vectors are in LDS at a time: 40 KB of vectors at most, and no more runs' worth of
// registers per thread than eight entries of each vector.
template <int E> constexpr int kScanRun = E == 16 ? 8 : 16;
// Whether a whole run's tokens are written out one after the other in the code (no loop): not where a
// lane already carries so many entries that more code in flight would not fit its registers.
template <int E> constexpr bool kScanUnrolled = E <= 8;

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ------------------------------------------------------------------ short convolution

// grid (tokens + items, ceil(channels / 256)). A token that lies taps - 1 or more behind its item's
// first token needs nothing but the step's own rows: one thread per (token, channel). The first
// taps - 1 tokens of an item read the inputs the state saved, and the state's saved inputs are
// replaced by the item's last ones: both are the work of one thread per (item, channel), so that
// nobody reads a saved input another thread has already replaced.
template <typename A, typename O>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const A* __restrict__ in, int64_t in_row, const float* __restrict__ w, const float* __restrict__ bias, O* __restrict__ out,
    int64_t out_row, float* __restrict__ state, int64_t state_row, const int32_t* __restrict__ tok_item,
    const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots, int tokens, int channels, int taps, int act) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int keep = taps - 1;
  const float* wc = w + static_cast<int64_t>(c) * taps;
  const float b = bias != nullptr ? bias[c] : 0.f;
  if (static_cast<int>(blockIdx.x) < tokens) {
    const int64_t t = blockIdx.x;
    const int64_t s0 = item_start[tok_item[t]];
    if (t - s0 < keep) return;
    float acc = b;
    for (int j = 0; j < taps; ++j) acc = fmaf(wc[j], to_float<A>(in[(t - keep + j) * in_row + c]), acc);
    out[t * out_row + c] = from_float<O>(act ? acc * sigmoidf_(acc) : acc);
    return;
  }
  const int item = static_cast<int>(blockIdx.x) - tokens;
  const int64_t s0 = item_start[item];
  const int n = static_cast<int>(item_start[item + 1] - s0);
  float* saved = state + static_cast<int64_t>(slots[item]) * state_row + c;      // saved[j * channels]: oldest first
  const int first = min(n, keep);
  for (int li = 0; li < first; ++li) {
    float acc = b;
    for (int j = 0; j < taps; ++j) {
      const int src = li - keep + j;
      const float v = src >= 0 ? to_float<A>(in[(s0 + src) * in_row + c]) : saved[static_cast<int64_t>(keep + src) * channels];
      acc = fmaf(wc[j], v, acc);
    }
    out[(s0 + li) * out_row + c] = from_float<O>(act ? acc * sigmoidf_(acc) : acc);
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

// grid (ceil(tokens / 4), heads), 256 threads: four tokens of one head, so that a row of the low-rank
// map's outer matrix is fetched once for four tokens. rows (activation type) hold r, k, v,
// the removal rate's logits (heads x dim each, at their columns) and the low-rank map's inner
// values (rank, at l_col). ops row = [r | k | v | w | p | c], heads x dim each, float:
//   w = exp(-decay_floor * sigmoid(sum_j w2[j, hc] tanh(l[j]) + w0[hc])), c = k / sqrt(sum k^2 + unit_eps),
//   p = -sigmoid(a + a_bias[hc]) * c. w2 is stored [rank][heads * dim].
constexpr int kPrepTokens = 4;

template <typename A>
__global__ __launch_bounds__(256) void general_delta_prepare_kernel(
    const A* __restrict__ rows, int64_t in_row, int r_col, int k_col, int v_col, int a_col, int l_col,
    const float* __restrict__ a_bias, const float* __restrict__ w2, const float* __restrict__ w0, float* __restrict__ ops,
    int64_t tokens, int heads, int dim, int rank, float decay_floor, float unit_eps) {
  extern __shared__ float prep_smem[];                 // tanh(l)[4][rank], then 1 / |k| of the four tokens
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kPrepTokens;
  const int nt = static_cast<int>(min(static_cast<int64_t>(kPrepTokens), tokens - t0));
  const int h = blockIdx.y;
  float* inv = prep_smem + kPrepTokens * rank;
  for (int idx = threadIdx.x; idx < nt * rank; idx += blockDim.x) {
    const int tk = idx / rank, j = idx - tk * rank;
    prep_smem[idx] = tanhf(to_float<A>(rows[(t0 + tk) * in_row + l_col + j]));
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  if (wave < nt) {
    const A* row = rows + (t0 + wave) * in_row + k_col + static_cast<int64_t>(h) * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += kWave) {
      const float k = to_float<A>(row[i]);
      ss = fmaf(k, k, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) inv[wave] = 1.f / sqrtf(ss + unit_eps);
  }
  __syncthreads();
  const int64_t hd = static_cast<int64_t>(heads) * dim;
  for (int idx = threadIdx.x; idx < nt * dim; idx += blockDim.x) {
    const int tk = idx / dim, i = idx - tk * dim;
    const A* row = rows + (t0 + tk) * in_row;
    const int64_t hc = static_cast<int64_t>(h) * dim + i;
    const float* w2c = w2 + hc;                          // column hc of the map stored [rank][heads * dim]: lanes read side by side
    const float* th = prep_smem + tk * rank;
    float low = w0[hc];
    for (int j = 0; j < rank; ++j) low = fmaf(w2c[j * hd], th[j], low);
    const float k = to_float<A>(row[k_col + hc]);
    const float c = k * inv[tk];
    float* o = ops + (t0 + tk) * 6 * hd + hc;
    o[0] = to_float<A>(row[r_col + hc]);
    o[hd] = k;
    o[2 * hd] = to_float<A>(row[v_col + hc]);
    o[3 * hd] = expf(-decay_floor * sigmoidf_(low));
    o[4 * hd] = -sigmoidf_(to_float<A>(row[a_col + hc]) + a_bias[hc]) * c;
    o[5 * hd] = c;
  }
}

// ------------------------------------------------------------------ the recurrence

// Sum over the 16 lanes of a row, in every lane, by four data-parallel moves inside the vector unit (lane
// pairs, pairs of pairs, the mirrored half row, the mirrored row) instead of four trips through LDS: the
// recurrence waits on this sum once per token.
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
  return v;
}

// One token's operands as a lane holds them while it walks: its E entries of the vectors, and the numbers.
// SAME (the gated rule: c = p = k, one decay number per head, the removal reads the decayed state) keeps
// k and r alone.
template <int E, bool SAME>
struct ScanToken {
  float k[E], r[E], c[SAME ? 1 : E], p[SAME ? 1 : E], d[SAME ? 1 : E];
  float ds, ps, xw, rp, rk;
};

template <int E, bool SAME>
__device__ __forceinline__ void scan_load(ScanToken<E, SAME>& t, const float* __restrict__ vec, const float* __restrict__ sca,
                                          const float* __restrict__ xs, int tk, int l, int col) {
  constexpr int DP = E * kLPC, NV = SAME ? 2 : 5;
  const float* v = vec + tk * NV * DP + l * E;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    t.k[e] = v[e];
    t.r[e] = v[DP + e];
    if constexpr (!SAME) {
      t.c[e] = v[2 * DP + e];
      t.p[e] = v[3 * DP + e];
      t.d[e] = v[4 * DP + e];
    }
  }
  const float* sc = sca + tk * 6;
  t.ds = sc[0];
  t.ps = sc[1];
  t.xw = sc[2] * xs[tk * kCols + col];
  t.rp = sc[3];
  t.rk = sc[4];
}

// One token: the column's E entries in s, the read-out returned (the same in all 16 lanes).
template <int E, bool SAME, bool RD, bool NR>
__device__ __forceinline__ float scan_step(const ScanToken<E, SAME>& t, float (&s)[E]) {
  if constexpr (NR) {
    // Nothing is taken out: S <- d S + k xw. The new column does not wait for a sum over the lanes;
    // only the read-out (r . d S) + xw (r . k) does, and nothing waits for that.
    float rd = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float dec = t.ds * s[e];
      rd = fmaf(t.r[e], dec, rd);
      s[e] = fmaf(t.k[e], t.xw, dec);
    }
    return fmaf(t.xw, t.rk, row16_sum(rd));
  }
  float dec[E];
  float dot = 0.f, rd = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    if constexpr (SAME) {
      dec[e] = t.ds * s[e];
      dot = fmaf(t.k[e], dec[e], dot);
    } else {
      dec[e] = t.d[e] * s[e];                            // the number per head is already in the vector
      dot = fmaf(t.c[e], RD ? dec[e] : s[e], dot);
    }
    rd = fmaf(t.r[e], dec[e], rd);
  }
  dot = row16_sum(dot);
  rd = row16_sum(rd);
  const float take = t.ps * dot;
  if constexpr (SAME) {
    const float w = take + t.xw;
#pragma unroll
    for (int e = 0; e < E; ++e) s[e] = fmaf(t.k[e], w, dec[e]);
    return fmaf(w, t.rk, rd);
  } else {
#pragma unroll
    for (int e = 0; e < E; ++e) s[e] = fmaf(t.k[e], t.xw, fmaf(t.p[e], take, dec[e]));
    return fmaf(t.xw, t.rk, fmaf(take, t.rp, rd));
  }
}

// Tokens tk and tk + 1 of a run of n: the next token's operands are read from LDS while one is computed.
// ta holds token tk on entry and token tk + 2 on exit.
template <int E, bool SAME, bool RD, bool NR>
__device__ __forceinline__ void scan_two(ScanToken<E, SAME>& ta, ScanToken<E, SAME>& tb, float (&s)[E], const float* __restrict__ vec,
                                         const float* __restrict__ sca, const float* __restrict__ xs, int tk, int n,
                                         float* __restrict__ o, int64_t out_row, int j, bool writes, int l, int col) {
  constexpr int TT = kScanRun<E>;
  scan_load(tb, vec, sca, xs, min(tk + 1, TT - 1), l, col);
  const float ra = scan_step<E, SAME, RD, NR>(ta, s);
  if (writes) o[tk * out_row + j] = ra;
  if (tk + 1 < n) {
    scan_load(ta, vec, sca, xs, min(tk + 2, TT - 1), l, col);
    const float rb = scan_step<E, SAME, RD, NR>(tb, s);
    if (writes) o[(tk + 1) * out_row + j] = rb;
  }
}

// grid (items, heads, ceil(vdim / 16)), 256 threads: column col = threadIdx.x / 16 of the block's 16,
// lane l of its 16 holds the E entries l * E .. l * E + E - 1 of the column (dim <= 16 E). The vectors
// of TT tokens at a time pass through LDS; the run after is already on its way from memory, in
// registers, while a run is walked, and a token's operands are read from LDS while the token before
// is computed. A token costs one dependent sum over the column: with dec = d * S and
// take = ps (c . S*), the new column is dec + p take + k xw, and its read-out r . S is
// (r . dec) + take (r . p) + xw (r . k), where r . dec is summed beside c . S* and the two
// products of vectors alone are formed once per token for all columns when the run arrives.
template <int E, bool SAME, bool RD, bool NR = false>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const float* __restrict__ kvec, const float* __restrict__ cvec, const float* __restrict__ pvec,
    const float* __restrict__ rvec, int64_t key_row, int heads_per_group, const float* __restrict__ dvec, int64_t dvec_row,
    const float* __restrict__ dscal, const float* __restrict__ pscal, const float* __restrict__ xscal, int64_t scal_row,
    const float* __restrict__ x, int64_t x_row, float* __restrict__ out, int64_t out_row, float* __restrict__ state,
    int64_t state_row, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots, int dim, int vdim) {
  constexpr int DP = E * kLPC;                          // the column's length, padded
  constexpr int TT = kScanRun<E>;                       // tokens per run
  constexpr int VPT = TT * DP / 256;                    // vector entries a thread carries per run
  constexpr int NV = SAME ? 2 : 5;                      // vectors per token in LDS: k, r (, c, p, d)
  constexpr int NS = 6;                                 // numbers per token: d, ps, xs, r . p, r . k
  __shared__ __align__(16) float vec[TT * NV * DP];
  __shared__ float sca[TT * NS];
  __shared__ float xs_[TT * kCols];
  const int item = blockIdx.x, h = blockIdx.y, g = h / heads_per_group;
  const int col = threadIdx.x / kLPC, l = threadIdx.x % kLPC;
  const int j0 = blockIdx.z * kCols, j = j0 + col;
  const int64_t s0 = item_start[item], s1 = item_start[item + 1];
  float* st = state + static_cast<int64_t>(slots[item]) * state_row + (static_cast<int64_t>(h) * vdim + j) * dim + l * E;
  float s[E];
#pragma unroll
  for (int e = 0; e < E; ++e) s[e] = (j < vdim && l * E + e < dim) ? st[e] : 0.f;

  float fk[VPT], fr[VPT], fc[SAME ? 1 : VPT], fp[SAME ? 1 : VPT], fd[SAME ? 1 : VPT], fx = 0.f, fs = 1.f;
  // Round tf fetches the run from token tf on into registers and walks the run before it, which the
  // round before fetched: the loads are in flight while the tokens are walked.
  for (int64_t tf = s0; tf < s1 + TT; tf += TT) {
    const int64_t t0 = tf - TT;                         // the run that is walked
    const int n = static_cast<int>(min(static_cast<int64_t>(TT), s1 - t0));
    if (tf > s0) {
      __syncthreads();                                  // everybody is done with the run before
#pragma unroll
      for (int u = 0; u < VPT; ++u) {
        const int idx = threadIdx.x + u * 256, tk = idx / DP, i = idx % DP;
        float* v = vec + tk * NV * DP + i;
        v[0] = fk[u];
        v[DP] = fr[u];
        if constexpr (!SAME) {
          v[2 * DP] = fc[u];
          v[3 * DP] = fp[u];
          v[4 * DP] = fd[u];
        }
      }
      if (threadIdx.x / kCols < TT) xs_[threadIdx.x] = fx;
      if (threadIdx.x < TT * 3) sca[(threadIdx.x / 3) * NS + threadIdx.x % 3] = fs;
      __syncthreads();
    }
    if (tf < s1) {
      const int m = static_cast<int>(min(static_cast<int64_t>(TT), s1 - tf));
#pragma unroll
      for (int u = 0; u < VPT; ++u) {
        const int idx = threadIdx.x + u * 256, tk = idx / DP, i = idx % DP;
        const bool in = tk < m && i < dim;
        const int64_t at = (tf + tk) * key_row + static_cast<int64_t>(g) * dim + i;
        fk[u] = in ? kvec[at] : 0.f;
        fr[u] = in ? rvec[at] : 0.f;
        if constexpr (!SAME) {
          fc[u] = in ? cvec[at] : 0.f;
          fp[u] = in ? pvec[at] : 0.f;
          float d = (in && dvec != nullptr) ? dvec[(tf + tk) * dvec_row + static_cast<int64_t>(h) * dim + i] : 1.f;
          if (in && dscal != nullptr) d *= dscal[(tf + tk) * scal_row + h];
          fd[u] = d;
        }
      }
      {
        const int tk = threadIdx.x / kCols, cc = threadIdx.x % kCols;
        fx = (tk < m && j0 + cc < vdim) ? x[(tf + tk) * x_row + static_cast<int64_t>(h) * vdim + j0 + cc] : 0.f;
      }
      if (threadIdx.x < TT * 3) {
        const int tk = threadIdx.x / 3, which = threadIdx.x % 3;
        const float* src = which == 0 ? dscal : which == 1 ? pscal : xscal;
        fs = (tk < m && src != nullptr) ? src[(tf + tk) * scal_row + h] : 1.f;
      }
    }
    if (tf == s0) continue;
    if (col < n) {                                      // r . p and r . k of token col, once for all columns
      const float* v = vec + col * NV * DP + l * E;
      float rp = 0.f, rk = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if constexpr (!SAME) rp = fmaf(v[DP + e], v[3 * DP + e], rp);
        rk = fmaf(v[DP + e], v[e], rk);
      }
      if constexpr (!SAME) rp = row16_sum(rp);
      rk = row16_sum(rk);
      if (l == 0) {
        sca[col * NS + 3] = rp;
        sca[col * NS + 4] = rk;
      }
    }
    __syncthreads();
    float* o = out + t0 * out_row + static_cast<int64_t>(h) * vdim;   // the same in every lane: the lane's part is j
    const bool writes = l == 0 && j < vdim;
    ScanToken<E, SAME> ta, tb;
    scan_load(ta, vec, sca, xs_, 0, l, col);
    if (kScanUnrolled<E> && n == TT) {                  // a whole run: every LDS address and row offset is a constant
#pragma unroll
      for (int tk = 0; tk < TT; tk += 2) scan_two<E, SAME, RD, NR>(ta, tb, s, vec, sca, xs_, tk, TT, o, out_row, j, writes, l, col);
    } else {
      for (int tk = 0; tk < n; tk += 2) scan_two<E, SAME, RD, NR>(ta, tb, s, vec, sca, xs_, tk, n, o, out_row, j, writes, l, col);
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

template <int E, bool SAME, bool RD, bool NR = false>
static int launch_delta_scan(hipStream_t s, dim3 grid, const float* kvec, const float* cvec, const float* pvec,
                             const float* rvec, int64_t key_row, int heads_per_group, const float* dvec, int64_t dvec_row,
                             const float* dscal, const float* pscal, const float* xscal, int64_t scal_row, const float* x,
                             int64_t x_row, float* out, int64_t out_row, float* state, int64_t state_row,
                             const int32_t* item_start, const int32_t* slots, int dim, int vdim) {
  delta_scan_kernel<E, SAME, RD, NR><<<grid, dim3(256), 0, s>>>(kvec, cvec, pvec, rvec, key_row, heads_per_group, dvec, dvec_row,
                                                           dscal, pscal, xscal, scal_row, x, x_row, out, out_row, state,
                                                           state_row, item_start, slots, dim, vdim);
  return check_launch("psamd_delta_scan");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_short_conv_to(void* stream, const void* in, int in_dtype, int64_t in_row, const float* taps_w, const float* bias,
                        void* out, int out_dtype, int64_t out_row, float* state, int64_t state_row, const int32_t* tok_item,
                        const int32_t* item_start, const int32_t* slots, int64_t tokens, int items, int channels, int taps,
                        int act) {
  PSAMD_REQUIRE(tokens >= 0 && items >= 0 && channels > 0 && taps >= 1 && taps <= kConvMaxTaps, "bad sizes (at most 16 taps)");
  PSAMD_REQUIRE(in_row >= channels && out_row >= channels && state_row >= static_cast<int64_t>(taps - 1) * channels,
                "rows too short");
  PSAMD_REQUIRE(tokens + items <= 2147483647LL && ceil_div(channels, 256) <= 65535, "too large for one launch");
  PSAMD_REQUIRE((in_dtype == kBF16 || in_dtype == kF32) && (out_dtype == kBF16 || out_dtype == kF32),
                "input and output are float32 or bfloat16");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens + items), static_cast<unsigned>(ceil_div(channels, 256)));
#define PSAMD_CONV(A_, O_)                                                                                              \
  short_conv_kernel<A_, O_><<<grid, dim3(256), 0, s>>>(static_cast<const A_*>(in), in_row, taps_w, bias,               \
                                                       static_cast<O_*>(out), out_row, state, state_row, tok_item,     \
                                                       item_start, slots, static_cast<int>(tokens), channels, taps, act)
  if (in_dtype == kBF16 && out_dtype == kF32) PSAMD_CONV(bf16_t, float);
  else if (in_dtype == kF32 && out_dtype == kF32) PSAMD_CONV(float, float);
  else if (in_dtype == kF32 && out_dtype == kBF16) PSAMD_CONV(float, bf16_t);
  else PSAMD_CONV(bf16_t, bf16_t);
#undef PSAMD_CONV
  return check_launch("psamd_short_conv");
}

int psamd_short_conv(void* stream, const void* in, int act_dtype, int64_t in_row, const float* taps_w, float* out,
                     int64_t out_row, float* state, int64_t state_row, const int32_t* tok_item, const int32_t* item_start,
                     const int32_t* slots, int64_t tokens, int items, int channels, int taps, int act) {
  return psamd_short_conv_to(stream, in, act_dtype, in_row, taps_w, nullptr, out, kF32, out_row, state, state_row, tok_item,
                             item_start, slots, tokens, items, channels, taps, act);
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
  PSAMD_REQUIRE(tokens <= 2147483647LL && heads <= 65535 && rank <= 3072, "too large for one launch (rank at most 3,072)");
  const int64_t hd = static_cast<int64_t>(heads) * dim;
  PSAMD_REQUIRE(std::max(std::max(r_col, k_col), std::max(v_col, a_col)) + hd <= in_row && l_col + rank <= in_row &&
                    std::min(std::min(std::min(r_col, k_col), std::min(v_col, a_col)), l_col) >= 0,
                "columns outside the rows");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(ceil_div(tokens, kPrepTokens)), static_cast<unsigned>(heads));
  const size_t smem = sizeof(float) * kPrepTokens * (static_cast<size_t>(rank) + 1);
  if (act_dtype == kBF16) {
    general_delta_prepare_kernel<bf16_t><<<grid, dim3(256), smem, s>>>(static_cast<const bf16_t*>(rows), in_row, r_col, k_col,
                                                                      v_col, a_col, l_col, a_bias, w2, w0, ops, tokens, heads,
                                                                      dim, rank, decay_floor, unit_eps);
  } else if (act_dtype == kF32) {
    general_delta_prepare_kernel<float><<<grid, dim3(256), smem, s>>>(static_cast<const float*>(rows), in_row, r_col, k_col,
                                                                     v_col, a_col, l_col, a_bias, w2, w0, ops, tokens, heads, dim,
                                                                     rank, decay_floor, unit_eps);
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
  const dim3 grid(static_cast<unsigned>(items), static_cast<unsigned>(heads), static_cast<unsigned>(ceil_div(vdim, kCols)));
  const int hpg = heads / key_groups;
  // The gated rule's form: one vector serves as key, direction and removal, the decay is a number per head.
  const bool same = cvec == kvec && pvec == kvec && dvec == nullptr && reads_decayed != 0;
  // reads_decayed 2: nothing is taken out (the removal's scale is zero throughout), in the gated rule's form only.
  PSAMD_REQUIRE(reads_decayed != 2 || same, "a recurrence without removal comes in the gated rule's form");
#define PSAMD_SCAN_ARGS                                                                                                   \
  s, grid, kvec, cvec, pvec, rvec, key_row, hpg, dvec, dvec_row, dscal, pscal, xscal, scal_row, x, x_row, out, out_row, state, \
      state_row, item_start, slots, dim, vdim
#define PSAMD_SCAN(E)                                                                                   \
  return same ? (reads_decayed == 2 ? launch_delta_scan<E, true, true, true>(PSAMD_SCAN_ARGS)           \
                                    : launch_delta_scan<E, true, true>(PSAMD_SCAN_ARGS))                \
              : reads_decayed ? launch_delta_scan<E, false, true>(PSAMD_SCAN_ARGS)                      \
                              : launch_delta_scan<E, false, false>(PSAMD_SCAN_ARGS)
  switch (e) {
    case 1: PSAMD_SCAN(1);
    case 2: PSAMD_SCAN(2);
    case 4: PSAMD_SCAN(4);
    case 8: PSAMD_SCAN(8);
    default: PSAMD_SCAN(16);
  }
#undef PSAMD_SCAN
#undef PSAMD_SCAN_ARGS
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
