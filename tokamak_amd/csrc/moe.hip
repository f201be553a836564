// Kernels of a routed feed-forward (a mixture of small gated experts) for gfx950.
//
// moe_route: per token the router's logits z = W_r h in float32, a score per expert
//   (sigmoid(z)), and the `top` experts with the largest scores (ties: the lower index) with
//   their scores as weights.
// moe_gate_up / moe_down: a block a
//   (token, chosen expert) pair and a slab of output channels; the pair's activation row sits in
//   LDS in float32, a wave walks eight weight rows at a time in 16-byte pieces.  The weight of a
//   chosen expert multiplies the expert's INPUT: since the first products are linear,
//   gate(w h) = w gate(h), the weight is applied to the two products in float32 before the
//   activation.  moe_down writes every pair's result to its own row of a float32 array
//   [top][tokens][width]; the kernel that reads it next (the norm that adds a sub-layer's output
//   to the stream) sums the `top` layers in order, so a token's result does not depend on what
//   else is in the step.
// moe_sort / moe_grouped, the form for many tokens in bfloat16: the (token, expert) pairs are
//   counted and listed expert by expert and cut into tiles of up to 64 pairs of one expert; a
//   block takes a tile and 128 or 256 output channels on the matrix cores (v_mfma_f32_16x16x32_bf16;
//   weights as operands straight from memory, activations too, or through LDS where K fills chunks
//   of 64), so an expert's weights are read once per tile of its tokens.  The second product writes every pair's result to its own row of a float32 array
//   [top][tokens][width], which the kernel that reads it next (the norm that adds a sub-layer's
//   output to the stream) sums in list order: no block adds into another's result.
//
// Router, scores, weights and every sum are float32 whatever the storage type.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

constexpr int kRouteWaves = 8;     // waves of a block of the router, which share a token's experts
constexpr int kRows = 8;           // weight rows a wave walks at once

template <typename T> struct Vec;
template <> struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// A block a token: its waves take the experts two at a time (lanes stride the width), then the
// first wave picks the largest scores.
//   correction (null or float32 [E]): the choice is made by score + correction, the weights are the
//     scores without it.
//   groups > 0: the experts form `groups` equal groups of neighbours; a group's score is the sum of its
//     two largest choice scores (of its one, if it has one expert); only experts of the `keep` groups
//     with the largest scores can be chosen (the others count as minus infinity).
//   normalise: the chosen experts' weights are divided by their sum (+ 1e-20); then all times `scale`.
template <typename T>
__global__ __launch_bounds__(kRouteWaves * kWave) void moe_route_kernel(
    const T* __restrict__ h, const float* __restrict__ router, int* __restrict__ chosen,
    float* __restrict__ weight, int N, int W, int E, int top, int softmax, const float* __restrict__ correction,
    int groups, int keep, int normalise, float scale) {
  extern __shared__ float score[];     // [E] scores, [E] choice scores, [groups] group scores
  float* choice = score + E;
  float* group_score = choice + E;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = blockIdx.x;
  const T* row = h + (size_t)n * W;
  constexpr int V = Vec<T>::N;
  const bool wide = W % V == 0 && (reinterpret_cast<uintptr_t>(h) % 16 == 0) && (reinterpret_cast<uintptr_t>(router) % 16 == 0);
  for (int e = 2 * wave; e < E; e += 2 * kRouteWaves) {
    // the sums run over k in the same order whichever path loads them
    const float* r0 = router + (size_t)e * W;
    const float* r1 = router + (size_t)min(e + 1, E - 1) * W;
    float a0 = 0.f, a1 = 0.f;
    if (wide) {
      for (int d = lane * V; d < W; d += kWave * V) {
        float x[V];
        Vec<T>::load(row + d, x);
#pragma unroll
        for (int i = 0; i < V; i += 4) {
          const float4 p = *reinterpret_cast<const float4*>(r0 + d + i), q = *reinterpret_cast<const float4*>(r1 + d + i);
          a0 = fmaf(x[i], p.x, a0); a0 = fmaf(x[i + 1], p.y, a0); a0 = fmaf(x[i + 2], p.z, a0); a0 = fmaf(x[i + 3], p.w, a0);
          a1 = fmaf(x[i], q.x, a1); a1 = fmaf(x[i + 1], q.y, a1); a1 = fmaf(x[i + 2], q.z, a1); a1 = fmaf(x[i + 3], q.w, a1);
        }
      }
    } else {
      for (int d = lane; d < W; d += kWave) {
        const float x = Elem<T>::load(row + d);
        a0 = fmaf(x, r0[d], a0);
        a1 = fmaf(x, r1[d], a1);
      }
    }
    a0 = wave_sum(a0);
    a1 = wave_sum(a1);
    if (lane == 0) {
      score[e] = softmax ? a0 : 1.f / (1.f + expf(-a0));
      if (e + 1 < E) score[e + 1] = softmax ? a1 : 1.f / (1.f + expf(-a1));
    }
  }
  __syncthreads();
  if (wave != 0) return;
  if (softmax) {
    // scores = softmax of the logits over all experts
    float top_z = -INFINITY;
    for (int e = lane; e < E; e += kWave) top_z = fmaxf(top_z, score[e]);
    top_z = wave_max(top_z);
    float sum = 0.f;
    for (int e = lane; e < E; e += kWave) sum += expf(score[e] - top_z);
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += kWave) score[e] = expf(score[e] - top_z) / sum;   // (a lane rewrites what it read)
    wave_lds_sync();
  }
  for (int e = lane; e < E; e += kWave) choice[e] = score[e] + (correction ? correction[e] : 0.f);
  wave_lds_sync();
  if (groups > 0) {
    const int size = E / groups;
    for (int g = lane; g < groups; g += kWave) {
      float first = -INFINITY, second = -INFINITY;
      for (int i = 0; i < size; ++i) {
        const float v = choice[g * size + i];
        if (v > first) { second = first; first = v; }
        else if (v > second) second = v;
      }
      group_score[g] = size > 1 ? first + second : first;
    }
    wave_lds_sync();
    // the `keep` best groups, one after the other; a kept group's score becomes +infinity
    for (int k = 0; k < keep; ++k) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += kWave) {
        const float v = group_score[g];
        if (v > best && v != INFINITY) { best = v; at = g; }
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) {
        const float ob = __shfl_xor(best, m, kWave);
        const int oa = __shfl_xor(at, m, kWave);
        if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
      }
      if (lane == 0 && at < groups) group_score[at] = INFINITY;
      wave_lds_sync();
    }
    for (int e = lane; e < E; e += kWave)
      if (group_score[e / size] != INFINITY) choice[e] = -INFINITY;
    wave_lds_sync();
  }
  // the largest `top` choice scores, one after the other; a lane looks at the experts lane, lane + 64, ...
  float total = 0.f;      // (lane 0's: the sum of the chosen experts' scores)
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += kWave) {
      const float v = choice[e];
      if (v > best) { best = v; at = e; }          // (ascending e: the lower index stays on ties)
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const float ob = __shfl_xor(best, m, kWave);
      const int oa = __shfl_xor(at, m, kWave);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (at >= E) at = 0;       // (fewer experts may be chosen than `top`: refused on the host, kept in range here)
    if (lane == 0) {
      chosen[(size_t)n * top + k] = at;
      weight[(size_t)n * top + k] = score[at];
      total += score[at];
      choice[at] = -INFINITY;
    }
    wave_lds_sync();
  }
  if (lane == 0 && (normalise || scale != 1.f)) {
    const float factor = normalise ? scale / (total + 1e-20f) : scale;
    for (int k = 0; k < top; ++k) weight[(size_t)n * top + k] *= factor;
  }
}

// a[p, c] = silu(w g) * (w u), g = Wg[e][c] . h[n], u = Wu[e][c] . h[n]; gate_up [E][2 F][W]
// (an expert's gate rows, then its up rows).  grid (pairs, slabs of channels).
// WIDE: rows are walked in 16-byte pieces (their length fills such pieces), else element by element.
template <typename T, bool WIDE>
__device__ __forceinline__ void load_piece(const T* p, float* o) {
  if constexpr (WIDE) Vec<T>::load(p, o);
  else o[0] = Elem<T>::load(p);
}

template <typename T, bool WIDE>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(
    const T* __restrict__ h, const T* __restrict__ gate_up, const int* __restrict__ chosen,
    const float* __restrict__ weight, T* __restrict__ act, int W, int F, int top, int slab, int on_output) {
  extern __shared__ float x[];         // [W]
  const int p = blockIdx.x, n = p / top;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  for (int d = threadIdx.x; d < W; d += blockDim.x) x[d] = Elem<T>::load(h + (size_t)n * W + d);
  __syncthreads();
  const int e = chosen[p];
  const float wt = weight[p];
  const T* wg = gate_up + (size_t)e * 2 * F * W;
  const T* wu = wg + (size_t)F * W;
  constexpr int V = WIDE ? Vec<T>::N : 1;
  const int c_end = min(F, (int)(blockIdx.y + 1) * slab);
  for (int c0 = blockIdx.y * slab + wave * kRows; c0 < c_end; c0 += nwaves * kRows) {
    float g[kRows], u[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) g[r] = u[r] = 0.f;
    for (int d = lane * V; d < W; d += kWave * V) {
      float xv[V];
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] = x[d + i];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const int c = min(c0 + r, F - 1);       // (a row past the end is walked again and not used)
        float a[V], b[V];
        load_piece<T, WIDE>(wg + (size_t)c * W + d, a);
        load_piece<T, WIDE>(wu + (size_t)c * W + d, b);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          g[r] = fmaf(a[i], xv[i], g[r]);
          u[r] = fmaf(b[i], xv[i], u[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      g[r] = wave_sum(g[r]);
      u[r] = wave_sum(u[r]);
    }
    if (lane < kRows && c0 + lane < c_end) {
      float gv = 0.f, uv = 0.f;
#pragma unroll
      for (int r = 0; r < kRows; ++r)
        if (r == lane) { gv = g[r]; uv = u[r]; }
      // the weight on the expert's input scales both first products; on its output it scales
      // the activations, which the second product carries through (it is linear)
      if (!on_output) gv *= wt;
      uv *= wt;
      Elem<T>::store(act + (size_t)p * F + c0 + lane, gv / (1.f + expf(-gv)) * uv);
    }
  }
}

// out[k][n][c] = Wd[e][c] . a[p] for the pair p = n top + k and its expert e; down [E][W][F]; out
// float32 [top][N][W], whose `top` layers the next kernel adds in order.  grid (pairs, slabs of columns).
constexpr int kDownRows = 16;      // weight rows a wave of the second product walks at once

template <typename T, bool WIDE>
__global__ __launch_bounds__(256) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ down, const int* __restrict__ chosen,
    float* __restrict__ out, int N, int W, int F, int top, int slab) {
  extern __shared__ float x[];         // [F]
  const int p = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  for (int d = threadIdx.x; d < F; d += blockDim.x) x[d] = Elem<T>::load(act + (size_t)p * F + d);
  __syncthreads();
  constexpr int V = WIDE ? Vec<T>::N : 1;
  const T* wd = down + (size_t)chosen[p] * W * F;
  float* dst = out + ((size_t)(p % top) * N + p / top) * W;
  const int c_end = min(W, (int)(blockIdx.y + 1) * slab);
  for (int c0 = blockIdx.y * slab + wave * kDownRows; c0 < c_end; c0 += nwaves * kDownRows) {
    float acc[kDownRows];
#pragma unroll
    for (int r = 0; r < kDownRows; ++r) acc[r] = 0.f;
    for (int d = lane * V; d < F; d += kWave * V) {
      float xv[V];
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] = x[d + i];
#pragma unroll
      for (int r = 0; r < kDownRows; ++r) {
        const int c = min(c0 + r, W - 1);
        float a[V];
        load_piece<T, WIDE>(wd + (size_t)c * F + d, a);
#pragma unroll
        for (int i = 0; i < V; ++i) acc[r] = fmaf(a[i], xv[i], acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < kDownRows; ++r) acc[r] = wave_sum(acc[r]);
    if (lane < kDownRows && c0 + lane < c_end) {
      float v = 0.f;
#pragma unroll
      for (int r = 0; r < kDownRows; ++r)
        if (r == lane) v = acc[r];
      dst[c0 + lane] = v;
    }
  }
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
union Frag8 {
  uint4 u;
  bf16x8 v;
};

constexpr int kTilePairs = 64;      // pairs of one expert a block takes
constexpr int kXcds = 8;            // dies of the GPU, each with an L2 of its own; blocks go to them in turn

// Which (tile, block of channels) a block of the one-dimensional grid takes.  Blocks are handed to
// the eight dies in turn, each die has an L2 of its own, and the tiles of one expert, which read
// the same weights, are neighbours in the tile list: so die d takes the d-th eighth of the work in
// order, tile fastest, and the tiles of an expert at one block of channels run on one die at about
// the same time and share the weights in its L2 (in plain grid order they land on different dies
// and every tile streams its expert's weights from memory again).  Measured (2,048 tokens over 16
// experts of the 8B shape, first product): plain order 0.34 PFLOP/s, this 0.41; groups of four
// tiles by all blocks of channels per die (so that a group's activations stay in L2 as well) 0.36.
__device__ __forceinline__ void tile_of_block(int tiles, int channel_blocks, int& tile, int& channels) {
  const int linear = blockIdx.x;
  const int per_die = gridDim.x / kXcds;                 // (tk_moe_grouped makes the grid a multiple of eight)
  const int work = (linear % kXcds) * per_die + linear / kXcds;
  tile = work < tiles * channel_blocks ? work % tiles : -1;
  channels = work / tiles;
}

constexpr int kSortThreads = 1024;

// One block: counts the pairs of every expert, lists the pairs expert by expert (order), and cuts
// every expert's list into tiles.  Which place a pair gets inside its expert's list depends on the
// order of LDS atomics; no result depends on it (a pair's products are its own).
__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(
    const int* __restrict__ chosen, int P, int E, int tile_pairs, int* __restrict__ order, int* __restrict__ tile_expert,
    int* __restrict__ tile_start, int* __restrict__ tile_count, int* __restrict__ num_tiles) {
  extern __shared__ int sort_lds[];     // count [E], first [E + 1], cursor [E]
  int* count = sort_lds;
  int* first = count + E;
  int* cursor = first + E + 1;
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      first[e] = at;
      for (int t = 0; t < count[e]; t += tile_pairs) {
        tile_expert[tiles] = e;
        tile_start[tiles] = at + t;
        tile_count[tiles] = min(tile_pairs, count[e] - t);
        ++tiles;
      }
      at += count[e];
    }
    first[E] = at;
    *num_tiles = tiles;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int e = chosen[p];
    order[first[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

// A block: tile blockIdx.x (up to 16 MT pairs of one expert) and four waves' output channels, a
// wave 32 of them (64 where there is no gate: as many products a load).  D[channel][pair] accumulates over K in steps of 32;
// lane (r, kb) holds the weights' row r and the pair r of a tile of 16, 8 consecutive k each.
// GATED: weights [E][2 R][K], an expert's gate rows then its up rows; a pair's activations are the
//   row of its token in x; out (bfloat16 [P][R]) = silu(w g) * (w u) with the pair's weight w.
// else: weights [E][R][K]; a pair's activations are its own row of x; out (float32
//   [top][N][R]) takes the pair (n, k)'s products at [k][n].
template <int MT, bool GATED>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ weights, const int* __restrict__ order,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_start, const int* __restrict__ tile_count,
    const int* __restrict__ num_tiles, const float* __restrict__ pair_weight, void* __restrict__ out,
    int N, int top, int R, int K, int max_tiles, int channel_blocks, int on_output) {
  int tile, channels;
  tile_of_block(max_tiles, channel_blocks, tile, channels);
  if (tile < 0 || tile >= *num_tiles) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int e = tile_expert[tile], start = tile_start[tile], cnt = tile_count[tile];
  constexpr int NT = GATED ? 2 : 4;             // tiles of 16 output channels a wave
  const int c0 = (channels * 4 + wave) * (16 * NT);
  if (c0 >= R) return;
  constexpr int WT = GATED ? 2 * NT : NT;       // weight fragments a step: gate and up, or down
  const bf16_t* base = weights + (size_t)e * (GATED ? 2 : 1) * R * K;
  const bf16_t* wp[WT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int row = min(c0 + t * 16 + r, R - 1);
    wp[t] = base + (size_t)row * K + kb * 8;
    if (GATED) wp[NT + t] = base + (size_t)(R + row) * K + kb * 8;
  }
  int pair[MT];
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    pair[t] = order[start + min(t * 16 + r, cnt - 1)];
    ap[t] = x + (size_t)(GATED ? pair[t] / top : pair[t]) * K + kb * 8;
  }
  float4v acc[WT][MT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  const int whole = K / 32;
  int s = 0;
  for (; s + 2 <= whole; s += 2) {
    Frag8 wf[2][WT], af[2][MT];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int t = 0; t < WT; ++t) wf[u][t].u = *reinterpret_cast<const uint4*>(wp[t] + (s + u) * 32);
#pragma unroll
      for (int t = 0; t < MT; ++t) af[u][t].u = *reinterpret_cast<const uint4*>(ap[t] + (s + u) * 32);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][i].v, af[u][j].v, acc[i][j], 0, 0, 0);
  }
  // leftover steps, the last of which may reach past K (K is a multiple of 8, so a 16-byte piece is
  // whole or absent; an absent piece is read at k = 0 and zeroed)
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (; s * 32 < K; ++s) {
    const bool kok = s * 32 + kb * 8 < K;
    const int koff = kok ? s * 32 : -kb * 8;
    Frag8 wf[WT], af[MT];
#pragma unroll
    for (int t = 0; t < WT; ++t) {
      const uint4 v = *reinterpret_cast<const uint4*>(wp[t] + koff);
      wf[t].u = kok ? v : zero;
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const uint4 v = *reinterpret_cast<const uint4*>(ap[t] + koff);
      af[t].u = kok ? v : zero;
    }
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, af[j].v, acc[i][j], 0, 0, 0);
  }

  // acc[i][j][q] = D[channel c0 + i * 16 + kb * 4 + q][pair j * 16 + r]
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (j * 16 + r >= cnt) continue;
    const int p = pair[j];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int c = c0 + i * 16 + kb * 4;
      if (c >= R) continue;
      if (GATED) {
        const float w = pair_weight[p];
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float g = on_output ? acc[i][j][q] : acc[i][j][q] * w, u = acc[NT + i][j][q] * w;
          v[q] = g / (1.f + expf(-g)) * u;
        }
        bf16_t* dst = reinterpret_cast<bf16_t*>(out) + (size_t)p * R + c;
        store_four<bf16_t>(dst, v[0], v[1], v[2], v[3], R - c, R % 4 == 0);
      } else {
        float* dst = reinterpret_cast<float*>(out) + ((size_t)(p % top) * N + p / top) * R + c;
        store_four<float>(dst, acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3], R - c, R % 4 == 0);
      }
    }
  }
}

// The same product where K is a multiple of 64: the tile's activations go through LDS, 64 k at a
// time, and are shared by the block's four waves (each reads its weights straight from memory as
// before), and the next chunk's operands are asked for before this chunk's products.  Measured on
// 8B-shaped experts (2,048 tokens, 16 experts, two a token): 227 TFLOP/s with operands straight from
// memory and no prefetch, 340 so; tiles of 128 pairs (twice the products a weight fragment, 252
// registers, two waves a SIMD instead of three) 310 and 257.
constexpr int kWideK = 64, kWideLd = kWideK + 8;   // (rows 144 bytes apart: 16-byte reads by row spread over the banks)

template <bool GATED, int ROWS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void moe_grouped_wide_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ weights, const int* __restrict__ order,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_start, const int* __restrict__ tile_count,
    const int* __restrict__ num_tiles, const float* __restrict__ pair_weight, void* __restrict__ out,
    int N, int top, int R, int K, int max_tiles, int channel_blocks, int on_output) {
  int tile, channels;
  tile_of_block(max_tiles, channel_blocks, tile, channels);
  if (tile < 0 || tile >= *num_tiles) return;
  __shared__ __attribute__((aligned(16))) bf16_t xs[ROWS * kWideLd];
  constexpr int MT = ROWS / 16;
  constexpr int XP = ROWS * 8 / 256;       // 16-byte pieces of a chunk that a thread copies
  constexpr int NT = GATED ? 2 : 4;
  constexpr int WT = 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int e = tile_expert[tile], start = tile_start[tile], cnt = tile_count[tile];
  const int c0 = (channels * 4 + wave) * (16 * NT);
  const bool active = c0 < R;          // (a wave past the last channel still copies its share of the activations)
  const bf16_t* base = weights + (size_t)e * (GATED ? 2 : 1) * R * K;
  const bf16_t* wp[WT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int row = min(c0 + t * 16 + r, R - 1);
    wp[t] = base + (size_t)row * K + kb * 8;
    if (GATED) wp[NT + t] = base + (size_t)(R + row) * K + kb * 8;
  }
  // the 16-byte pieces of a chunk of activations that this thread copies: piece i * 256 + tid is
  // (row, eighth of the chunk's k) = (piece / 8, piece % 8)
  const bf16_t* xp[XP];
  int xat[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int piece = i * 256 + tid, row = piece >> 3, part = piece & 7;
    const int p = order[start + min(row, cnt - 1)];
    xp[i] = x + (size_t)(GATED ? p / top : p) * K + part * 8;
    xat[i] = row * kWideLd + part * 8;
  }
  float4v acc[WT][MT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // the next chunk's operands are asked for before this chunk's products, so that memory and the
  // matrix cores work side by side
  uint4 xa[XP], xn[XP];
  Frag8 wf[2][WT], wn[2][WT];
#pragma unroll
  for (int i = 0; i < XP; ++i) xa[i] = *reinterpret_cast<const uint4*>(xp[i]);
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < WT; ++t) wf[u][t].u = *reinterpret_cast<const uint4*>(wp[t] + u * 32);
  for (int k0 = 0; k0 < K; k0 += kWideK) {
    __syncthreads();      // every wave has read the chunk before
#pragma unroll
    for (int i = 0; i < XP; ++i) *reinterpret_cast<uint4*>(xs + xat[i]) = xa[i];
    __syncthreads();
    const int k1 = k0 + kWideK < K ? k0 + kWideK : k0;     // (past the end: the same chunk again, not used)
#pragma unroll
    for (int i = 0; i < XP; ++i) xn[i] = *reinterpret_cast<const uint4*>(xp[i] + k1);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < WT; ++t) wn[u][t].u = *reinterpret_cast<const uint4*>(wp[t] + k1 + u * 32);
    if (active) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          Frag8 af;
          af.u = *reinterpret_cast<const uint4*>(xs + (j * 16 + r) * kWideLd + u * 32 + kb * 8);
#pragma unroll
          for (int i = 0; i < WT; ++i)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][i].v, af.v, acc[i][j], 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < XP; ++i) xa[i] = xn[i];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < WT; ++t) wf[u][t].u = wn[u][t].u;
  }
  if (!active) return;
  // acc[i][j][q] = D[channel c0 + i * 16 + kb * 4 + q][pair j * 16 + r]
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (j * 16 + r >= cnt) continue;
    const int p = order[start + j * 16 + r];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int c = c0 + i * 16 + kb * 4;
      if (c >= R) continue;
      if (GATED) {
        const float w = pair_weight[p];
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float g = on_output ? acc[i][j][q] : acc[i][j][q] * w, u = acc[NT + i][j][q] * w;
          v[q] = g / (1.f + expf(-g)) * u;
        }
        bf16_t* dst = reinterpret_cast<bf16_t*>(out) + (size_t)p * R + c;
        store_four<bf16_t>(dst, v[0], v[1], v[2], v[3], R - c, R % 4 == 0);
      } else {
        float* dst = reinterpret_cast<float*>(out) + ((size_t)(p % top) * N + p / top) * R + c;
        store_four<float>(dst, acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3], R - c, R % 4 == 0);
      }
    }
  }
}

}  // namespace

// h [N, W] in dtype; router [E, W] float32; chosen [N, top] int32 and weight [N, top] float32 out
// softmax: the scores are the softmax of the logits over all experts, else their sigmoids
TK_API int tk_moe_route(int dtype, const void* h, const float* router, int* chosen, float* weight, int N,
                        int W, int E, int top, int softmax, const float* correction, int groups, int keep,
                        int normalise, float scale, hipStream_t stream) {
  if (N <= 0) return 0;
  if (E < 1 || top < 1 || top > E || W < 1 || (size_t)E * 12 > 60 * 1024) return -1;
  if (groups < 0 || (groups > 0 && (E % groups != 0 || keep < 1 || keep > groups || (long)keep * (E / groups) < top))) return -1;
  const unsigned blocks = (unsigned)N;
  const size_t lds = ((size_t)2 * E + (size_t)groups) * sizeof(float);
  if (dtype == 0)
    moe_route_kernel<float><<<blocks, kRouteWaves * kWave, lds, stream>>>((const float*)h, router, chosen, weight, N, W, E, top, softmax,
                                                                         correction, groups, keep, normalise, scale);
  else
    moe_route_kernel<bf16_t><<<blocks, kRouteWaves * kWave, lds, stream>>>((const bf16_t*)h, router, chosen, weight, N, W, E, top, softmax,
                                                                          correction, groups, keep, normalise, scale);
  return launch_status();
}

static int slab_for(int channels, long rows) {
  // slabs of channels so that some 1,024 blocks exist, each at least a turn of its four waves
  const long want = (1024 + rows - 1) / rows;
  long slab = (channels + want - 1) / want;
  slab = (slab + 4 * kRows - 1) / (4 * kRows) * (4 * kRows);
  return (int)(slab < 4 * kRows ? 4 * kRows : slab);
}

// act[N * top, F] = silu(w gate) * (w up) of every (token, chosen expert) pair
// on_output: act = w * silu(gate) * up instead (the weight acts on the expert's output)
TK_API int tk_moe_gate_up(int dtype, const void* h, const void* gate_up, const int* chosen, const float* weight,
                          void* act, int N, int W, int F, int top, int on_output, hipStream_t stream) {
  if (N <= 0) return 0;
  const bool wide = W % (dtype == 0 ? 4 : 8) == 0;
  if ((size_t)W * 4 > 96 * 1024 || (long)N * top > 0x7fffffffL / 2) return -1;
  const int slab = slab_for(F, (long)N * top);
  const dim3 grid(N * top, (F + slab - 1) / slab);
  const size_t lds = (size_t)W * sizeof(float);
#define TK_GU(T_, WIDE_)                                                                               \
  {                                                                                                    \
    static bool allowed = false;                                                                       \
    if (!allowed) {                                                                                    \
      const hipError_t err = hipFuncSetAttribute((const void*)moe_gate_up_kernel<T_, WIDE_>,           \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
      if (err != hipSuccess) return (int)err;                                                          \
      allowed = true;                                                                                  \
    }                                                                                                  \
    moe_gate_up_kernel<T_, WIDE_><<<grid, 256, lds, stream>>>((const T_*)h, (const T_*)gate_up, chosen, weight, \
                                                              (T_*)act, W, F, top, slab, on_output);   \
  }
  if (dtype == 0 && wide) TK_GU(float, true)
  else if (dtype == 0) TK_GU(float, false)
  else if (wide) TK_GU(bf16_t, true)
  else TK_GU(bf16_t, false)
#undef TK_GU
  return launch_status();
}

// out[top][N][W] float32: layer k holds down[e] act[pair] of every token's k-th chosen expert
TK_API int tk_moe_down(int dtype, const void* act, const void* down, const int* chosen, float* out, int N, int W,
                       int F, int top, hipStream_t stream) {
  if (N <= 0) return 0;
  const bool wide = F % (dtype == 0 ? 4 : 8) == 0;
  if ((size_t)F * 4 > 96 * 1024) return -1;
  const long want = (1024 + (long)N * top - 1) / ((long)N * top);
  long slab = (W + want - 1) / want;
  slab = (slab + 4 * kDownRows - 1) / (4 * kDownRows) * (4 * kDownRows);
  const dim3 grid(N * top, (unsigned)((W + slab - 1) / slab));
  const size_t lds = (size_t)F * sizeof(float);
#define TK_DN(T_, WIDE_)                                                                               \
  {                                                                                                    \
    static bool allowed = false;                                                                       \
    if (!allowed) {                                                                                    \
      const hipError_t err = hipFuncSetAttribute((const void*)moe_down_kernel<T_, WIDE_>,              \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
      if (err != hipSuccess) return (int)err;                                                          \
      allowed = true;                                                                                  \
    }                                                                                                  \
    moe_down_kernel<T_, WIDE_><<<grid, 256, lds, stream>>>((const T_*)act, (const T_*)down, chosen, out, N, W, F, top, \
                                                           (int)slab);                                 \
  }
  if (dtype == 0 && wide) TK_DN(float, true)
  else if (dtype == 0) TK_DN(float, false)
  else if (wide) TK_DN(bf16_t, true)
  else TK_DN(bf16_t, false)
#undef TK_DN
  return launch_status();
}

// The pairs of `chosen` [P] listed expert by expert and cut into tiles of up to tile_pairs (64):
// order [P], tile_expert / tile_start / tile_count [P / tile_pairs + E], num_tiles [1].
TK_API int tk_moe_sort(const int* chosen, int P, int E, int tile_pairs, int* order, int* tile_expert, int* tile_start,
                       int* tile_count, int* num_tiles, hipStream_t stream) {
  if (P <= 0) return 0;
  if (E < 1 || (size_t)(3 * E + 1) * 4 > 60 * 1024 || tile_pairs != kTilePairs) return -1;
  moe_sort_kernel<<<1, kSortThreads, (size_t)(3 * E + 1) * sizeof(int), stream>>>(chosen, P, E, tile_pairs, order, tile_expert,
                                                                                 tile_start, tile_count, num_tiles);
  return launch_status();
}

// bfloat16 only.  gated != 0: x [N][K] the tokens' rows, weights [E][2 R][K], out bfloat16 [N top][R];
// gated == 2: as gated, but out = w * silu(g) * u (the pair's weight acts on the expert's output, which the
// second product, being linear, carries through).
// gated == 0: x [N top][K] the pairs' rows, weights [E][R][K], out float32 [top][N][R].
// max_tiles: the length of the tile lists (blocks past num_tiles leave at once).
TK_API int tk_moe_grouped(int gated, const void* x, const void* weights, const int* order, const int* tile_expert,
                          const int* tile_start, const int* tile_count, const int* num_tiles, const float* pair_weight,
                          void* out, int N, int top, int R, int K, int max_tiles, int rows_hint, int tile_pairs,
                          hipStream_t stream) {
  if (N <= 0 || max_tiles <= 0) return 0;
  if (K % 8 != 0 || K < 8 || R < 1 || (uintptr_t)x % 16 != 0 || (uintptr_t)weights % 16 != 0) return -1;
  const int channels = gated ? 128 : 256;      // a block's
  const int channel_blocks = (R + channels - 1) / channels;
  const int total_blocks = max_tiles * channel_blocks;
  const dim3 grid((total_blocks + kXcds - 1) / kXcds * kXcds);      // (see tile_of_block)
  if (tile_pairs != kTilePairs) return -1;
  if (K % kWideK == 0 && rows_hint > 32) {
    // whole chunks of 64 k: the tile's activations through LDS, the next chunk asked for ahead
#define TK_WIDE(GATED_, ROWS_)                                                                                     \
  moe_grouped_wide_kernel<GATED_, ROWS_><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)weights, order, \
                                                                   tile_expert, tile_start, tile_count, num_tiles, \
                                                                   pair_weight, out, N, top, R, K, max_tiles,      \
                                                                   channel_blocks, gated == 2)
    if (gated) TK_WIDE(true, 64);
    else TK_WIDE(false, 64);
#undef TK_WIDE
    return launch_status();
  }
#define TK_GROUPED(MT_)                                                                                           \
  {                                                                                                               \
    if (gated)                                                                                                    \
      moe_grouped_kernel<MT_, true><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)weights, order,    \
                                                              tile_expert, tile_start, tile_count, num_tiles,     \
                                                              pair_weight, out, N, top, R, K, max_tiles,          \
                                                              channel_blocks, gated == 2);                        \
    else                                                                                                          \
      moe_grouped_kernel<MT_, false><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)weights, order,   \
                                                               tile_expert, tile_start, tile_count, num_tiles,    \
                                                               pair_weight, out, N, top, R, K, max_tiles,         \
                                                               channel_blocks, 0);                                \
  }
  // rows_hint: the most pairs an expert can have (the step's pairs): tiles are never fuller than that
  if (rows_hint <= 16) TK_GROUPED(1)
  else if (rows_hint <= 32) TK_GROUPED(2)
  else TK_GROUPED(4)
#undef TK_GROUPED
  return launch_status();
}

TK_SLOTS(tk_moe_route)
TK_SLOTS(tk_moe_gate_up)
TK_SLOTS(tk_moe_down)
TK_SLOTS(tk_moe_sort)
TK_SLOTS(tk_moe_grouped)
