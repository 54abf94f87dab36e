// Mixture-of-experts feed-forward: the router, and the experts in two forms.
//
// * Pair by pair: one (token, choice) pair per workgroup row, the expert's matrices read once per
//   pair. It is the form of the 32-bit path at every size (templated on the element type, sums in
//   float, in an order that does not depend on the step) and of bfloat16 steps of one or two tokens.
// * Grouped (bfloat16): the step's pairs are sorted by expert, and every expert's pairs go through
//   its matrices in tiles of 16 or 64 pairs on the matrix cores (v_mfma_f32_16x16x32_bf16), so an
//   expert is read once per tile of pairs instead of once per pair: a decode batch reads each
//   expert it uses once, a prompt's portion runs as grouped products.
//
// Router: z = x . w_r[e] (+ bias[e]) in float; the `top` largest are taken, the lower index among
// equals. mode 0: the score is sigmoid(z) and is the weight as it is; mode 1: the weights are the
// softmax over the chosen z alone. Expert: with h = weight * x, g = min(gate h, limit), u = clamp(up h,
// -limit, limit), act = g * sigmoid(gate_alpha * g) * (u + up_shift), out = down act. There the weight
// multiplies the expert's input, so it cannot be pulled out of the clamps; with weight_on_output the
// expert sees x itself and the weight multiplies out (limit = infinity, gate_alpha = 1, up_shift = 0
// then make the plain SiLU-gated expert).

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// Dot product of a row of n elements with a float vector in LDS, dealt out over the 64 lanes;
// every lane returns the whole sum. bfloat16 rows whose length is a multiple of 8 are read in
// 16-byte pieces.
template <typename W>
__device__ __forceinline__ float wave_dot(const W* __restrict__ row, const float* __restrict__ xs, int n, int lane) {
  float acc = 0.f;
  if (sizeof(W) == 2 && (n & 7) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int chunks = n >> 3;
    for (int c = lane; c < chunks; c += kWave) {
      const uint4 q = *reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(row) + 8 * c);
      const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
      const float* xp = xs + 8 * c;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc = fmaf(__uint_as_float(w4[i] << 16), xp[2 * i], acc);
        acc = fmaf(__uint_as_float(w4[i] & 0xffff0000u), xp[2 * i + 1], acc);
      }
    }
  } else if (sizeof(W) == 4 && (n & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int chunks = n >> 2;
    float acc2 = 0.f;
    for (int c = lane; c < chunks; c += 2 * kWave) {
      const int c2 = c + kWave;
      const float4 q = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(row) + 4 * c);
      const float4 q2 = c2 < chunks ? *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(row) + 4 * c2)
                                    : float4{0.f, 0.f, 0.f, 0.f};
      const float* xp = xs + 4 * c;
      const float* xp2 = xs + 4 * min(c2, chunks - 1);
      acc = fmaf(q.x, xp[0], acc); acc = fmaf(q.y, xp[1], acc); acc = fmaf(q.z, xp[2], acc); acc = fmaf(q.w, xp[3], acc);
      acc2 = fmaf(q2.x, xp2[0], acc2); acc2 = fmaf(q2.y, xp2[1], acc2); acc2 = fmaf(q2.z, xp2[2], acc2); acc2 = fmaf(q2.w, xp2[3], acc2);
    }
    acc += acc2;
  } else {
    for (int i = lane; i < n; i += kWave) acc = fmaf(to_float<W>(row[i]), xs[i], acc);
  }
  return wave_sum(acc);
}

// ------------------------------------------------------------------ router

// The router's choice for one token by one wave: score[] (LDS, `experts` entries: sigmoid(z) in mode
// 0, z in mode 1) -> chosen / weight [top], largest first, the lower index among equals; taken
// entries are overwritten. Mode 1 then turns the chosen z into their softmax.
__device__ __forceinline__ void pick_top(float* score, int experts, int top, int mode, int32_t* __restrict__ chosen,
                                         float* __restrict__ weight, int lane) {
  const float kTaken = -__builtin_inff();
  for (int j = 0; j < top; ++j) {
    float best = kTaken;
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += kWave) {
      const float s = score[e];
      if (s > best) {                                    // ascending e: the first of equals stays
        best = s;
        at = e;
      }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (lane == 0) {
      chosen[j] = at;
      weight[j] = best;
      if (at != 0x7fffffff) score[at] = kTaken;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if (mode == 1 && lane == 0) {
    const float m = weight[0];                           // the largest comes first
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += expf(weight[j] - m);
    for (int j = 0; j < top; ++j) weight[j] = expf(weight[j] - m) / sum;
  }
}

__device__ __forceinline__ float router_score(float z, const float* __restrict__ bias, int e, int mode) {
  if (bias != nullptr) z += bias[e];
  return mode == 0 ? 1.f / (1.f + expf(-z)) : z;
}

// One block of four waves per token: the waves share the experts' dot products, then wave 0
// picks the `top` largest scores one after the other (each pick: a strided scan and a wave
// reduction that prefers the lower index among equals).
template <typename A>
__global__ __launch_bounds__(256) void moe_route_kernel(const A* __restrict__ x, const float* __restrict__ w_router,
                                                        int32_t* __restrict__ chosen, float* __restrict__ weight,
                                                        int K, int experts, int top, const float* __restrict__ bias, int mode) {
  extern __shared__ __align__(16) float route_smem[];    // xs[K], score[experts]
  float* xs = route_smem;
  float* score = route_smem + K;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < K; i += blockDim.x) xs[i] = to_float<A>(x[t * K + i]);
  __syncthreads();
  for (int e = wave; e < experts; e += 4) {
    const float z = wave_dot<float>(w_router + static_cast<int64_t>(e) * K, xs, K, lane);
    if (lane == 0) score[e] = router_score(z, bias, e, mode);
  }
  __syncthreads();
  if (wave != 0) return;
  pick_top(score, experts, top, mode, chosen + t * top, weight + t * top, lane);
}

// The same choice from logits a product has already written (z[t, :] float). One wave per token,
// four tokens per block.
__global__ __launch_bounds__(256) void moe_topk_kernel(const float* __restrict__ z, int32_t* __restrict__ chosen,
                                                       float* __restrict__ weight, int64_t tokens, int experts, int top,
                                                       const float* __restrict__ bias, int mode) {
  extern __shared__ __align__(16) float topk_smem[];     // score[4][experts]
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  if (t >= tokens) return;
  float* score = topk_smem + wave * experts;
  for (int e = lane; e < experts; e += kWave) score[e] = router_score(z[t * experts + e], bias, e, mode);
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
  pick_top(score, experts, top, mode, chosen + t * top, weight + t * top, lane);
}

// ------------------------------------------------------------------ experts, pair by pair

constexpr int kRowsPerWave = 4;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;

// grid (pairs, ceil(F / 16)): the block stages h = weight * x[t] in LDS and each wave computes
// kRowsPerWave activations of the pair's expert.
template <typename A>
__global__ __launch_bounds__(256) void moe_gate_up_rows_kernel(
    const A* __restrict__ x, const int32_t* __restrict__ chosen, const float* __restrict__ weight,
    const A* __restrict__ w_gate_up, A* __restrict__ act, int K, int F, int experts, int top, float gate_alpha,
    float limit, float up_shift, int weight_on_output) {
  extern __shared__ __align__(16) float rows_smem[];     // h[K]
  const int64_t pair = blockIdx.x;
  const int64_t t = pair / top;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int e = min(max(chosen[pair], 0), experts - 1);
  const float wgt = weight_on_output ? 1.f : weight[pair];
  for (int i = threadIdx.x; i < K; i += blockDim.x) rows_smem[i] = wgt * to_float<A>(x[t * K + i]);
  __syncthreads();
  const A* we = w_gate_up + static_cast<int64_t>(e) * 2 * F * K;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int f = static_cast<int>(blockIdx.y) * kRowsPerBlock + wave * kRowsPerWave + r;
    if (f >= F) break;
    float g = wave_dot<A>(we + static_cast<int64_t>(f) * K, rows_smem, K, lane);
    float u = wave_dot<A>(we + static_cast<int64_t>(F + f) * K, rows_smem, K, lane);
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    if (lane == 0) act[pair * F + f] = from_float<A>(g / (1.f + expf(-gate_alpha * g)) * (u + up_shift));
  }
}

// grid (pairs, ceil(K / 16)): out[j][t][k] = down[e][k] . act[pair].
template <typename A>
__global__ __launch_bounds__(256) void moe_down_rows_kernel(
    const A* __restrict__ act, const int32_t* __restrict__ chosen, const A* __restrict__ w_down,
    float* __restrict__ out, int64_t tokens, int K, int F, int experts, int top, const float* __restrict__ out_weight) {
  extern __shared__ __align__(16) float rows_smem[];     // act[F]
  const int64_t pair = blockIdx.x;
  const int64_t t = pair / top;
  const int j = static_cast<int>(pair - t * top);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int e = min(max(chosen[pair], 0), experts - 1);
  for (int i = threadIdx.x; i < F; i += blockDim.x) rows_smem[i] = to_float<A>(act[pair * F + i]);
  __syncthreads();
  const A* we = w_down + static_cast<int64_t>(e) * K * F;
  float* o = out + (static_cast<int64_t>(j) * tokens + t) * K;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int k = static_cast<int>(blockIdx.y) * kRowsPerBlock + wave * kRowsPerWave + r;
    if (k >= K) break;
    const float v = wave_dot<A>(we + static_cast<int64_t>(k) * F, rows_smem, F, lane);
    if (lane == 0) o[k] = out_weight != nullptr ? out_weight[pair] * v : v;
  }
}


// ------------------------------------------------------------------ experts, grouped by expert

// One workgroup sorts the step's pairs by expert and lists the tiles of `tile_rows` pairs the
// products run over. ints: sorted[pairs] (pair indices, expert by expert), then per tile slot
// tile_expert, tile_first (index into sorted), tile_count; slots past the last tile hold -1.
// The order of an expert's pairs among themselves is whatever the atomics gave: every pair's
// result is computed from its own row alone, so it does not matter which rows share a tile.
// `count`, `start`, `tstart`, `cursor` are LDS arrays of `experts` integers each.
__device__ __forceinline__ void group_pairs(const int32_t* __restrict__ chosen, int pairs, int experts, int tile_rows,
                                            int max_tiles, int32_t* __restrict__ sorted, int32_t* __restrict__ tile_expert,
                                            int32_t* __restrict__ tile_first, int32_t* __restrict__ tile_count,
                                            int32_t* count, int32_t* start, int32_t* tstart, int32_t* cursor,
                                            int32_t* n_tiles) {
  for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&count[min(max(chosen[p], 0), experts - 1)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < experts; ++e) {
      start[e] = at;
      tstart[e] = nt;
      at += count[e];
      nt += (count[e] + tile_rows - 1) / tile_rows;
    }
    *n_tiles = min(nt, max_tiles);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    int nt = tstart[e];
    for (int r0 = 0; r0 < count[e] && nt < max_tiles; r0 += tile_rows, ++nt) {
      tile_expert[nt] = e;
      tile_first[nt] = start[e] + r0;
      tile_count[nt] = min(tile_rows, count[e] - r0);
    }
  }
  for (int nt = *n_tiles + threadIdx.x; nt < max_tiles; nt += blockDim.x) tile_expert[nt] = -1;
  for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
    const int e = min(max(chosen[p], 0), experts - 1);
    sorted[start[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* __restrict__ chosen, int pairs, int experts,
                                                         int tile_rows, int max_tiles, int32_t* __restrict__ sorted,
                                                         int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_first,
                                                         int32_t* __restrict__ tile_count) {
  extern __shared__ int32_t group_smem[];      // count, start, tstart, cursor [experts] each, n_tiles
  group_pairs(chosen, pairs, experts, tile_rows, max_tiles, sorted, tile_expert, tile_first, tile_count, group_smem,
              group_smem + experts, group_smem + 2 * experts, group_smem + 3 * experts, group_smem + 4 * experts);
}

// The choice from logits and the sorting in one workgroup of 16 waves, for steps of so few tokens
// that one workgroup does the choice at once (a decode step): a wave per token, then the sorting above.
__global__ __launch_bounds__(1024) void moe_topk_group_kernel(const float* __restrict__ z, int32_t* __restrict__ chosen,
                                                              float* __restrict__ weight, int tokens, int experts, int top,
                                                              int tile_rows, int max_tiles, int32_t* __restrict__ sorted,
                                                              int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_first,
                                                              int32_t* __restrict__ tile_count, const float* __restrict__ bias,
                                                              int mode) {
  extern __shared__ int32_t group_smem[];      // as above, then score[16][experts]
  float* score = reinterpret_cast<float*>(group_smem + 4 * experts + 1) + (threadIdx.x >> 6) * experts;
  const int lane = threadIdx.x & (kWave - 1);
  for (int t = threadIdx.x >> 6; t < tokens; t += 16) {
    for (int e = lane; e < experts; e += kWave) score[e] = router_score(z[static_cast<int64_t>(t) * experts + e], bias, e, mode);
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    pick_top(score, experts, top, mode, chosen + t * top, weight + t * top, lane);
  }
  __threadfence_block();
  __syncthreads();                             // the workgroup's own writes of `chosen` are read below
  group_pairs(chosen, tokens * top, experts, tile_rows, max_tiles, sorted, tile_expert, tile_first, tile_count, group_smem,
              group_smem + experts, group_smem + 2 * experts, group_smem + 3 * experts, group_smem + 4 * experts);
}

constexpr int kGroupBK = 64;                   // k per staging round
constexpr int kGroupLD = kGroupBK + 8;         // LDS row stride of the staged pairs, in elements

// One workgroup (4 waves) per (64 * RT output columns, tile of MT * 16 pairs of one expert). The
// pairs' input rows pass through LDS 64 k at a time (gathered through `sorted`). GATED: the
// pair's weight on the expert's input is applied to the float32 sums, gate (w x) = w (gate x),
// before the clamps: the same number without a rounding of w x, and no arithmetic while staging
// (scaling and rounding the rows there cost as many vector cycles as the matrix instructions). Every
// wave streams its 16 * RT rows of the expert's matrix from memory (GATED: gate rows and the up
// rows that belong to them) and multiplies them with all MT tiles of pairs. The next round's
// rows of both operands are asked for before the current round is multiplied (registers, then
// the other of two LDS buffers), so one barrier per round is all the waves wait for.
//   GATED: out_act[pair][n] = act(gate, up) in bfloat16, N = F columns, w = [E][2N][K].
//   else:  out_f32[(pair % top) * tokens + pair / top][n] = sum, N = hidden columns, w = [E][N][K],
//          rows of `a` are indexed by pair.
template <int MT, int RT, bool GATED>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const bf16_t* __restrict__ a, const float* __restrict__ pair_weight, const bf16_t* __restrict__ w,
    const int32_t* __restrict__ sorted, const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_first,
    const int32_t* __restrict__ tile_count, bf16_t* __restrict__ out_act, float* __restrict__ out_f32, int64_t tokens,
    int K, int N, int top, float gate_alpha, float limit, float up_shift) {
  constexpr int ROWS = MT * 16;
  constexpr int PIECES = ROWS * (kGroupBK / 8);              // 16-byte pieces of a round's pairs
  constexpr int PPT = (PIECES + 255) / 256;                  // pieces per thread
  constexpr int KK = kGroupBK / 32;
  __shared__ __align__(16) bf16_t as[2][ROWS * kGroupLD];
  __shared__ int32_t pair_s[ROWS];
  const int slot = blockIdx.y;
  const int e = tile_expert[slot];
  if (e < 0) return;                            // uniform for the workgroup
  const int first = tile_first[slot], count = tile_count[slot];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = (static_cast<int>(blockIdx.x) * 4 + wave) * 16 * RT;     // this wave's first column
  if (threadIdx.x < ROWS) pair_s[threadIdx.x] = threadIdx.x < count ? sorted[first + threadIdx.x] : -1;
  const bf16_t* wg[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int nrow = min(n0 + rt * 16 + r, N - 1);
    wg[rt] = w + (static_cast<int64_t>(e) * (GATED ? 2 : 1) * N + nrow) * K + 8 * g;
  }
  const int64_t up_off = static_cast<int64_t>(N) * K;                      // GATED: from a gate row to its up row
  f32x4 acc_g[RT][MT], acc_u[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc_g[rt][mt] = acc_u[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();

  // This thread's pieces of a round: which pair's row, where from, its weight.
  const bf16_t* src[PPT];
#pragma unroll
  for (int p = 0; p < PPT; ++p) {
    const int idx = static_cast<int>(threadIdx.x) + p * 256;
    const int row = min(idx, PIECES - 1) / (kGroupBK / 8), c = min(idx, PIECES - 1) % (kGroupBK / 8);
    const int pair = pair_s[row];
    src[p] = (pair >= 0 && idx < PIECES) ? a + static_cast<int64_t>(GATED ? pair / top : pair) * K + 8 * c : nullptr;
  }
  uint4 areg[PPT];
  bf16x8 wa[KK][RT], wb[KK][RT];
  auto ask = [&](int k0) {                       // the round's rows of both operands, into registers
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
      const int c8 = 8 * ((static_cast<int>(threadIdx.x) + p * 256) % (kGroupBK / 8));
      areg[p] = (src[p] != nullptr && k0 + c8 < K) ? *reinterpret_cast<const uint4*>(src[p] + k0) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int k = k0 + kk * 32;
      const bool in = k + 8 * g < K;            // K is a multiple of 8: a piece is inside or outside as a whole
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int i = 0; i < 8; ++i) wa[kk][rt][i] = wb[kk][rt][i] = static_cast<__bf16>(0.f);
        if (in) {
          wa[kk][rt] = *reinterpret_cast<const bf16x8*>(wg[rt] + k);
          if (GATED) wb[kk][rt] = *reinterpret_cast<const bf16x8*>(wg[rt] + up_off + k);
        }
      }
    }
  };
  auto stage = [&](int buf) {                    // the pairs' pieces from registers into LDS
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
      const int idx = static_cast<int>(threadIdx.x) + p * 256;
      if (idx >= PIECES) continue;
      *reinterpret_cast<uint4*>(as[buf] + (idx / (kGroupBK / 8)) * kGroupLD + 8 * (idx % (kGroupBK / 8))) = areg[p];
    }
  };
  ask(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += kGroupBK, buf ^= 1) {
    bf16x8 ca[KK][RT], cb[KK][RT];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        ca[kk][rt] = wa[kk][rt];
        cb[kk][rt] = wb[kk][rt];
      }
    const bool more = k0 + kGroupBK < K;
    if (more) ask(k0 + kGroupBK);               // in flight while this round is multiplied
    // The pairs' operand of every step is read from LDS two steps ahead of the matrix instructions
    // that use it (read right in front of them, every group of four waited for its operand first).
    const bf16_t* bsrc = as[buf] + r * kGroupLD + 8 * g;
    auto b_of = [&](int step) {
      return *reinterpret_cast<const bf16x8*>(bsrc + (step % MT) * 16 * kGroupLD + (step / MT) * 32);
    };
    bf16x8 bq[3];
    bq[0] = b_of(0);
    if (KK * MT > 1) bq[1] = b_of(1);
#pragma unroll
    for (int step = 0; step < KK * MT; ++step) {
      const int kk = step / MT, mt = step % MT;
      if (step + 2 < KK * MT) bq[(step + 2) % 3] = b_of(step + 2);
      __builtin_amdgcn_sched_barrier(0);        // the read stays in front of this step's matrix instructions
      const bf16x8 b = bq[step % 3];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        acc_g[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ca[kk][rt], b, acc_g[rt][mt], 0, 0, 0);
        if (GATED) acc_u[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cb[kk][rt], b, acc_u[rt][mt], 0, 0, 0);
      }
    }
    if (more) stage(buf ^ 1);                   // nobody reads that buffer: all passed the last barrier after reading it
    __syncthreads();
  }
  // Lane (r, g) holds, for the pair in row mt * 16 + r, the four columns n0 + rt * 16 + 4 g .. + 3.
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int pair = pair_s[mt * 16 + r];
    if (pair < 0) continue;
    const float pw = pair_weight != nullptr ? pair_weight[pair] : 1.f;   // on the input's sums (GATED) or on the output's
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int nc = n0 + rt * 16 + 4 * g;
      if (GATED) {
        bf16_t* o = out_act + static_cast<int64_t>(pair) * N + nc;
        bf16_t res[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float gg = fminf(pw * acc_g[rt][mt][v], limit);
          const float uu = fminf(fmaxf(pw * acc_u[rt][mt][v], -limit), limit);
          res[v] = float_to_bf16(gg / (1.f + __expf(-gate_alpha * gg)) * (uu + up_shift));
        }
        if (nc + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<ushort4*>(o) = ushort4{res[0], res[1], res[2], res[3]};
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (nc + v < N) o[v] = res[v];
        }
      } else {
        float* o = out_f32 + (static_cast<int64_t>(pair % top) * tokens + pair / top) * N + nc;
        if (nc + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<float4*>(o) = float4{pw * acc_g[rt][mt][0], pw * acc_g[rt][mt][1], pw * acc_g[rt][mt][2], pw * acc_g[rt][mt][3]};
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (nc + v < N) o[v] = pw * acc_g[rt][mt][v];
        }
      }
    }
  }
}

template <int MT, int RT>
static int launch_grouped(hipStream_t s, const void* x, const float* weight, const void* w_gate_up, const void* w_down,
                          void* act, float* out, const int32_t* ints, int max_tiles, int64_t tokens, int K, int F, int top,
                          float gate_alpha, float limit, float up_shift, int weight_on_output) {
  const int64_t pairs = tokens * top;
  const int32_t* sorted = ints;
  const int32_t* t_e = ints + pairs;
  const int32_t* t_f = t_e + max_tiles;
  const int32_t* t_c = t_f + max_tiles;
  moe_grouped_kernel<MT, RT, true><<<dim3(static_cast<unsigned>(ceil_div(F, 64 * RT)), static_cast<unsigned>(max_tiles)), dim3(256), 0, s>>>(
      static_cast<const bf16_t*>(x), weight_on_output ? nullptr : weight, static_cast<const bf16_t*>(w_gate_up), sorted, t_e, t_f, t_c,
      static_cast<bf16_t*>(act), nullptr, tokens, K, F, top, gate_alpha, limit, up_shift);
  if (check_launch("psamd_moe_experts_grouped (gate/up)")) return 1;
  moe_grouped_kernel<MT, RT, false><<<dim3(static_cast<unsigned>(ceil_div(K, 64 * RT)), static_cast<unsigned>(max_tiles)), dim3(256), 0, s>>>(
      static_cast<const bf16_t*>(act), weight_on_output ? weight : nullptr, static_cast<const bf16_t*>(w_down), sorted, t_e, t_f, t_c, nullptr, out,
      tokens, F, K, top, 0.f, 0.f, 0.f);
  return check_launch("psamd_moe_experts_grouped (down)");
}

template <typename A>
static int launch_experts_rows(hipStream_t s, const void* x, const int32_t* chosen, const float* weight,
                               const void* w_gate_up, const void* w_down, void* act, float* out, int64_t tokens, int K,
                               int F, int experts, int top, float gate_alpha, float limit, float up_shift,
                               int weight_on_output) {
  const unsigned pairs = static_cast<unsigned>(tokens * top);
  moe_gate_up_rows_kernel<A><<<dim3(pairs, static_cast<unsigned>(ceil_div(F, kRowsPerBlock))), dim3(256),
                               sizeof(float) * K, s>>>(
      static_cast<const A*>(x), chosen, weight, static_cast<const A*>(w_gate_up), static_cast<A*>(act), K, F, experts, top,
      gate_alpha, limit, up_shift, weight_on_output);
  if (check_launch("psamd_moe_experts_rows (gate/up)")) return 1;
  moe_down_rows_kernel<A><<<dim3(pairs, static_cast<unsigned>(ceil_div(K, kRowsPerBlock))), dim3(256), sizeof(float) * F,
                            s>>>(static_cast<const A*>(act), chosen, static_cast<const A*>(w_down), out, tokens, K, F,
                                 experts, top, weight_on_output ? weight : nullptr);
  return check_launch("psamd_moe_experts_rows (down)");
}

// out[t, :] *= sigmoid(x[t] . w): one number per token on the output of a branch every token takes.
// One workgroup per token, the dot product in float.
template <typename A>
__global__ __launch_bounds__(256) void row_gate_kernel(float* __restrict__ out, const A* __restrict__ x,
                                                       const float* __restrict__ w, int out_hidden, int hidden) {
  __shared__ float parts[4];
  const int64_t t = blockIdx.x;
  float acc = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) acc = fmaf(to_float<A>(x[t * hidden + i]), w[i], acc);
  const float g = 1.f / (1.f + expf(-block_sum(acc, parts, 4)));
  float* o = out + t * out_hidden;
  for (int i = threadIdx.x; i < out_hidden; i += 256) o[i] *= g;
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_moe_grouped_tile_rows(int64_t pairs, int experts);
int psamd_moe_grouped_max_tiles(int64_t pairs, int experts);

int psamd_moe_route(void* stream, const void* x, int x_dtype, const float* w_router, int32_t* chosen, float* weight,
                    int64_t tokens, int K, int experts, int top, const float* bias, int mode) {
  PSAMD_REQUIRE(mode == 0 || mode == 1, "router mode 0 (sigmoid scores) or 1 (softmax over the chosen)");
  PSAMD_REQUIRE(tokens >= 0 && K > 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * (static_cast<size_t>(K) + experts) <= 64 * 1024, "row and scores do not fit in LDS");
  PSAMD_REQUIRE(tokens <= 2147483647LL, "too many tokens for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t smem = sizeof(float) * (static_cast<size_t>(K) + experts);
  const dim3 grid(static_cast<unsigned>(tokens));
  if (x_dtype == kBF16) {
    moe_route_kernel<bf16_t><<<grid, dim3(256), smem, s>>>(static_cast<const bf16_t*>(x), w_router, chosen, weight, K,
                                                          experts, top, bias, mode);
  } else if (x_dtype == kF32) {
    moe_route_kernel<float><<<grid, dim3(256), smem, s>>>(static_cast<const float*>(x), w_router, chosen, weight, K,
                                                         experts, top, bias, mode);
  } else {
    return fail("psamd_moe_route: x must be float32 or bfloat16");
  }
  return check_launch("psamd_moe_route");
}

int psamd_moe_topk(void* stream, const float* logits, int32_t* chosen, float* weight, int64_t tokens, int experts,
                   int top, const float* bias, int mode) {
  PSAMD_REQUIRE(mode == 0 || mode == 1, "router mode 0 (sigmoid scores) or 1 (softmax over the chosen)");
  PSAMD_REQUIRE(tokens >= 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * 4 * static_cast<size_t>(experts) <= 64 * 1024, "scores do not fit in LDS");
  PSAMD_REQUIRE(ceil_div(tokens, 4) <= 2147483647LL, "too many tokens for one launch");
  if (tokens == 0) return 0;
  moe_topk_kernel<<<dim3(static_cast<unsigned>(ceil_div(tokens, 4))), dim3(256), sizeof(float) * 4 * experts,
                    static_cast<hipStream_t>(stream)>>>(logits, chosen, weight, tokens, experts, top, bias, mode);
  return check_launch("psamd_moe_topk");
}

int psamd_moe_topk_group(void* stream, const float* logits, int32_t* chosen, float* weight, int32_t* ints, int64_t tokens,
                         int experts, int top, const float* bias, int mode) {
  PSAMD_REQUIRE(mode == 0 || mode == 1, "router mode 0 (sigmoid scores) or 1 (softmax over the chosen)");
  PSAMD_REQUIRE(tokens >= 1 && tokens <= 64 && experts > 0 && experts <= 1024 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(ints != nullptr, "the grouping needs its integer scratch");
  const int64_t pairs = tokens * top;
  const int rows = psamd_moe_grouped_tile_rows(pairs, experts);
  const int max_tiles = psamd_moe_grouped_max_tiles(pairs, experts);
  moe_topk_group_kernel<<<dim3(1), dim3(1024), sizeof(int32_t) * (4 * experts + 1) + sizeof(float) * 16 * experts,
                          static_cast<hipStream_t>(stream)>>>(logits, chosen, weight, static_cast<int>(tokens), experts, top, rows,
                                                              max_tiles, ints, ints + pairs, ints + pairs + max_tiles,
                                                              ints + pairs + 2 * max_tiles, bias, mode);
  return check_launch("psamd_moe_topk_group");
}

int psamd_moe_experts_rows(void* stream, const void* x, const int32_t* chosen, const float* weight,
                           const void* w_gate_up, const void* w_down, void* act, float* out, int dtype,
                           int64_t tokens, int K, int F, int experts, int top, float gate_alpha, float limit,
                           float up_shift, int weight_on_output) {
  PSAMD_REQUIRE(tokens >= 0 && K > 0 && F > 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * static_cast<size_t>(std::max(K, F)) <= 64 * 1024, "a row does not fit in LDS");
  PSAMD_REQUIRE(tokens * top <= 2147483647LL && ceil_div(std::max(K, F), kRowsPerBlock) <= 65535, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kBF16)
    return launch_experts_rows<bf16_t>(s, x, chosen, weight, w_gate_up, w_down, act, out, tokens, K, F, experts, top,
                                       gate_alpha, limit, up_shift, weight_on_output);
  if (dtype == kF32)
    return launch_experts_rows<float>(s, x, chosen, weight, w_gate_up, w_down, act, out, tokens, K, F, experts, top,
                                      gate_alpha, limit, up_shift, weight_on_output);
  return fail("psamd_moe_experts_rows: dtype must be float32 or bfloat16");
}

// Pairs per tile of the grouped form for a step of this many pairs over this many experts: 128 when
// the experts have at least twice that many pairs each on average (an expert's last tile is half
// empty on average: 512 tokens of 8 choices over 32 experts took 204 us in tiles of 128, one full
// and one nearly empty per expert), 64 from 48 pairs per expert on, 16 below.
int psamd_moe_grouped_tile_rows(int64_t pairs, int experts) {
  return pairs >= 256LL * experts ? 128 : (pairs >= 48LL * experts ? 64 : 16);
}

// Tile slots the grouped form's grid has for such a step (every expert may end in a tile that is not full).
int psamd_moe_grouped_max_tiles(int64_t pairs, int experts) {
  const int rows = psamd_moe_grouped_tile_rows(pairs, experts);
  return static_cast<int>(std::min<int64_t>(ceil_div(pairs, rows) + experts, pairs));
}

int psamd_moe_experts_grouped(void* stream, const void* x, const int32_t* chosen, const float* weight,
                              const void* w_gate_up, const void* w_down, void* act, float* out, int32_t* ints,
                              int64_t tokens, int K, int F, int experts, int top, float gate_alpha, float limit,
                              float up_shift, int grouped_already, int weight_on_output) {
  PSAMD_REQUIRE(tokens >= 0 && K > 0 && F > 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(K % 8 == 0 && F % 8 == 0, "K and F must be multiples of 8");
  PSAMD_REQUIRE(experts <= 4096 && tokens * top <= (1 << 24), "too many experts or pairs");
  PSAMD_REQUIRE(ints != nullptr, "the grouping needs its integer scratch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t pairs = tokens * top;
  const int rows = psamd_moe_grouped_tile_rows(pairs, experts);
  const int max_tiles = psamd_moe_grouped_max_tiles(pairs, experts);
  PSAMD_REQUIRE(max_tiles <= 65535, "too many tiles for one launch");
  if (grouped_already == 0) {
    moe_group_kernel<<<dim3(1), dim3(1024), sizeof(int32_t) * (4 * experts + 1), s>>>(
        chosen, static_cast<int>(pairs), experts, rows, max_tiles, ints, ints + pairs, ints + pairs + max_tiles,
        ints + pairs + 2 * max_tiles);
    if (check_launch("psamd_moe_experts_grouped (grouping)")) return 1;
  }
  if (rows == 128)
    return launch_grouped<8, 2>(s, x, weight, w_gate_up, w_down, act, out, ints, max_tiles, tokens, K, F, top, gate_alpha,
                                limit, up_shift, weight_on_output);
  if (rows == 64)
    return launch_grouped<4, 2>(s, x, weight, w_gate_up, w_down, act, out, ints, max_tiles, tokens, K, F, top, gate_alpha,
                                limit, up_shift, weight_on_output);
  return launch_grouped<1, 1>(s, x, weight, w_gate_up, w_down, act, out, ints, max_tiles, tokens, K, F, top, gate_alpha, limit,
                              up_shift, weight_on_output);
}

int psamd_row_gate(void* stream, float* out, const void* x, int act_dtype, const float* w, int64_t tokens, int out_hidden,
                   int hidden) {
  PSAMD_REQUIRE(tokens >= 0 && out_hidden > 0 && hidden > 0 && tokens <= 2147483647LL, "bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens));
  if (act_dtype == kBF16) {
    row_gate_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(out, static_cast<const bf16_t*>(x), w, out_hidden, hidden);
  } else if (act_dtype == kF32) {
    row_gate_kernel<float><<<grid, dim3(256), 0, s>>>(out, static_cast<const float*>(x), w, out_hidden, hidden);
  } else {
    return fail("psamd_row_gate: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_row_gate");
}

}  // extern "C"
