// Kernels of a selective state-space mixer with a scalar decay per head (gfx950).
//
// The mixer's input projection yields, per token, [z | x | B | C | dt].
//
// conv_silu: x, B and C together pass a short causal convolution per channel, a bias and SiLU:
//     u_t[c] = silu(b[c] + sum_j w[c][j] in_(t - (taps - 1) + j)[c]),  j = 0 .. taps - 1,
//   the last tap meeting the token itself.  The inputs of the taps - 1 positions before a step's first
//   token come from the request's state (zeros before the sequence's start), which then takes the
//   step's last inputs (conv_carry, or the same kernel where a request's tokens are one segment).
// ssd_scan: per (request, head), over the step's tokens in order,
//     dt = softplus(dt_in + dt_bias),  S <- exp(-exp(A_log) dt) S + dt B_t x_t^T,  y_t = S^T C_t + D x_t
//   with the state S [state, vdim] in float32 registers (a thread owns a few state rows of one value
//   column); head h reads the B and C of group h / (heads / groups).
// gated_group_norm: y * silu(z), divided by its root mean square over each of `norm_groups` equal parts
//   of the row, times a weight.
//
// Step sizes, decays with their exponentials, the recurrence, its state, the gate's product and the
// norm are float32 whatever the storage type; x, B and C enter as the convolution stored them.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

constexpr int kMaxTaps = 8;
constexpr int kConvSegment = 64;   // tokens of a request that one thread of the convolution walks
constexpr int kScanTokens = 8;     // tokens staged in LDS at a time by the scan

// an input of [rows, ld] elements: T, or float32, or `parts` float32 partial sums `stride` elements apart
struct SsmIn {
  const void* p;
  int f32;
  int parts;
  long stride;
};

template <typename T>
__device__ __forceinline__ float load_in(const SsmIn& in, size_t idx) {
  if (!in.f32) return Elem<T>::load(reinterpret_cast<const T*>(in.p) + idx);
  const float* f = reinterpret_cast<const float*>(in.p) + idx;
  float s = f[0];
  int i = 1;
  for (; i + 3 < in.parts; i += 4) {      // four loads in flight; the sums in the order of the parts
    const float a = f[(size_t)i * in.stride], b = f[(size_t)(i + 1) * in.stride];
    const float c = f[(size_t)(i + 2) * in.stride], d = f[(size_t)(i + 3) * in.stride];
    s = (((s + a) + b) + c) + d;
  }
  for (; i < in.parts; ++i) s += f[(size_t)i * in.stride];
  return s;
}

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// grid (channel blocks, requests, segments of kConvSegment tokens).  proj rows are ld long, the
// convolution's channels start at column col0.  state: float32 [slots][taps - 1][C], oldest first.
template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(
    SsmIn proj, long ld, int col0, const float* __restrict__ w, const float* __restrict__ bias,
    float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
    T* __restrict__ out, int C, int taps, int update) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int req = blockIdx.y;
  const int first = q_start[req], end = q_start[req + 1];
  const int t_lo = first + blockIdx.z * kConvSegment, t_hi = min(end, t_lo + kConvSegment);
  if (c >= C || t_lo >= end) return;
  float* st = taps > 1 ? state + (size_t)state_slots[req] * (taps - 1) * C + c : nullptr;
  // taps and window sit at the END of arrays of kMaxTaps: index kMaxTaps - 1 is the token itself
  float wv[kMaxTaps], win[kMaxTaps];
#pragma unroll
  for (int k = 0; k < kMaxTaps; ++k) {
    const int j = k - (kMaxTaps - taps);
    wv[k] = j >= 0 ? w[(size_t)c * taps + j] : 0.f;
    win[k] = 0.f;
  }
#pragma unroll
  for (int d = 1; d < kMaxTaps; ++d) {
    if (d < taps) {
      const int local = t_lo - first - d;     // the input d positions before the segment's first token
      win[kMaxTaps - d] = local >= 0 ? load_in<T>(proj, (size_t)(t_lo - d) * ld + col0 + c)
                                     : st[(size_t)(taps - 1 + local) * C];
    }
  }
  const float b = bias[c];
  for (int t = t_lo; t < t_hi; ++t) {
#pragma unroll
    for (int k = 0; k < kMaxTaps - 1; ++k) win[k] = win[k + 1];
    win[kMaxTaps - 1] = load_in<T>(proj, (size_t)t * ld + col0 + c);
    float acc = b;
#pragma unroll
    for (int k = 0; k < kMaxTaps; ++k) acc = fmaf(wv[k], win[k], acc);
    Elem<T>::store(out + (size_t)t * C + c, silu(acc));
  }
  if (update) {      // (the request's tokens are this one segment: the window now ends at its last token)
#pragma unroll
    for (int k = 1; k < kMaxTaps; ++k) {
      const int j = k - (kMaxTaps - (taps - 1));
      if (j >= 0) st[(size_t)j * C] = win[k];
    }
  }
}

// The state after a step: the last taps - 1 inputs of every request, from the step's rows or, where the
// step brought fewer, from the state before it.  A thread a (request, channel): it reads what it needs, then writes.
template <typename T>
__global__ __launch_bounds__(256) void conv_carry_kernel(
    SsmIn proj, long ld, int col0, float* __restrict__ state, const int* __restrict__ q_start,
    const int* __restrict__ state_slots, int C, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int req = blockIdx.y;
  if (c >= C) return;
  const int first = q_start[req], count = q_start[req + 1] - first;
  float* st = state + (size_t)state_slots[req] * (taps - 1) * C + c;
  float keep[kMaxTaps - 1];
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j) {
    keep[j] = 0.f;
    if (j < taps - 1) {
      const int local = count - (taps - 1) + j;
      keep[j] = local >= 0 ? load_in<T>(proj, (size_t)(first + local) * ld + col0 + c) : st[(size_t)(taps - 1 + local) * C];
    }
  }
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j)
    if (j < taps - 1) st[(size_t)j * C] = keep[j];
}

// Sums over the KS neighbouring lanes that share a column group, for the COUNT values v[0 .. COUNT) that
// every lane holds: at each step a lane keeps one half of its values and hands the other half to the lane
// M away, which keeps that half (the lane whose bit M is set keeps the upper one), so that the numbers
// that travel halve from step to step (31 exchanges for 32 values over 32 lanes, where summing every value
// over all lanes takes 160).  Afterwards lane ks holds, in v[0 .. max(COUNT / KS, 1)), the complete sums of
// the values from index ks * COUNT / KS on (with more lanes than values: of value ks / (KS / COUNT), in
// every lane of that run).
template <int COUNT, int M>
__device__ __forceinline__ void sum_and_deal(float (&v)[32], int ks) {
  if constexpr (M >= 1) {
    if constexpr (COUNT > 1) {
      constexpr int H = COUNT / 2;
      const bool upper = (ks & M) != 0;
#pragma unroll
      for (int i = 0; i < H; ++i) {
        const float send = upper ? v[i] : v[i + H];
        const float keep = upper ? v[i + H] : v[i];
        v[i] = keep + __shfl_xor(send, M, kWave);
      }
      sum_and_deal<H, M / 2>(v, ks);
    } else {
      v[0] += __shfl_xor(v[0], M, kWave);
      sum_and_deal<1, M / 2>(v, ks);
    }
  }
}

struct ScanShape {
  int heads, groups, ns, vdim;      // ns: the state's size per value channel
  int columns;                      // groups of four value columns that a block holds
  int slices;                       // threads that share a column group, each with RS rows of the state (a power of two)
};

// A block a (request, head, share of the value columns).  u: the convolution's output [N, C] = [x | B | C].
// dt_in: rows ld long, the heads' step sizes from column dt_col.  y: float32 [N, heads * vdim].
//
// A thread owns RS rows by four columns of the state in registers, so that the 16-byte pieces of dt B
// and C it reads from LDS for a token serve four columns each (a thread that owns one column reads a
// B and a C for every multiply-add pair, and the kernel is then bound by LDS reads: 1.78 -> 1.07 ms for
// 2,048 tokens of 128 heads of 128 x 64).  The KS threads that share a column group are neighbouring
// lanes of one wave: the outputs of a round's eight tokens are summed over them with lane exchanges
// (sum_and_deal: no LDS array, no barrier), and every lane writes the sums it is left with.
//
// Long portions are cut into chunks of `chunk` tokens that run side by side (the decay is one number a
// head and token, so a chunk's effect on the state is S_end = P S_start + L with P the product of its
// decays and L its end state from zeros):
//   MODE 1: a block a (request, chunk, head, share): from zeros to L and P, no output;
//   ssd_chunk_starts_kernel: per request the chunks in order, S_start of each, the request's new state;
//   MODE 2: the same blocks again, each from its S_start, with the outputs.
// MODE 0 walks a request's tokens in one block from the request's state.  A chunk's place in the scratch
// arrays is its number among all chunks of the step (requests in order).
template <typename T, int RS, int KS, int MODE>
__global__ __launch_bounds__(1024) void ssd_scan_kernel(
    const T* __restrict__ u, int C, SsmIn dt_in, long ld, int dt_col, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ skip, float* __restrict__ state,
    const int* __restrict__ q_start, const int* __restrict__ state_slots, float* __restrict__ y, ScanShape sh,
    int chunk, int max_chunks, float* __restrict__ chunk_state, float* __restrict__ chunk_decay) {
  constexpr int TB = kScanTokens, CS = 4;
  constexpr int nsp = KS * RS;       // rows with the padding (zeros behind ns)
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* bb = lds;                   // [TB][nsp]: dt B
  float* cc = bb + TB * nsp;         // [TB][nsp]: C
  float* aa = cc + TB * nsp;         // [TB]: the decay
  const int ns = sh.ns, vdim = sh.vdim;
  const int req = MODE == 0 ? blockIdx.x : blockIdx.x / max_chunks, head = blockIdx.y;
  int first = q_start[req];
  int end = q_start[req + 1];
  size_t place = 0;       // of this chunk in the scratch arrays
  if (MODE != 0) {
    const int ci = blockIdx.x % max_chunks;
    if (first + ci * chunk >= end) return;      // (the whole block, before any barrier)
    int before = 0;
    for (int r = 0; r < req; ++r) before += (q_start[r + 1] - q_start[r] + chunk - 1) / chunk;
    place = (size_t)(before + ci) * sh.heads + head;
    first += ci * chunk;
    end = min(end, first + chunk);
  }
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int ks = tid & (KS - 1), jl = tid / KS;
  const int j0 = (blockIdx.z * sh.columns + jl) * CS;       // the thread's first value column
  const bool owns = jl < sh.columns && j0 < vdim;           // (threads that only fill the last wave own nothing)
  const int k0 = ks * RS;
  const int inner = sh.heads * vdim;
  const int group = head / (sh.heads / sh.groups);
  const int b_col = inner + group * ns, c_col = inner + sh.groups * ns + group * ns;
  // a head's state lies as [groups of four columns][ns rows][4]: a thread's rows are one run of 16-byte
  // pieces, and the threads of a column group (neighbouring lanes) read neighbouring runs
  const size_t head_elems = (size_t)((vdim + 3) / 4) * ns * 4;
  float* S = (MODE == 0 ? state + ((size_t)state_slots[req] * sh.heads + head) * head_elems
                        : chunk_state + place * head_elems) + ((size_t)(j0 >> 2) * ns + k0) * 4;
  float s[RS][CS];
#pragma unroll
  for (int r = 0; r < RS; ++r) {
    float4 row = make_float4(0.f, 0.f, 0.f, 0.f);
    if (MODE != 1 && owns && k0 + r < ns) row = *reinterpret_cast<const float4*>(S + r * 4);
    s[r][0] = row.x; s[r][1] = row.y; s[r][2] = row.z; s[r][3] = row.w;
  }
  const float rate = expf(a_log[head]), bias = dt_bias[head], d_skip = skip[head];
  float decayed = 1.f;      // the product of the chunk's decays (MODE 1)

  for (int t0 = first; t0 < end; t0 += TB) {
    const int tb = min(TB, end - t0);
    for (int i = tid; i < tb * nsp; i += nthreads) {
      const int t = i / nsp, n = i - t * nsp;
      const size_t row = (size_t)(t0 + t) * C;
      // (every element forms its token's step size itself: the same float32 operations, no barrier for it)
      const float dt = softplus(load_in<T>(dt_in, (size_t)(t0 + t) * ld + dt_col + head) + bias);
      bb[i] = n < ns ? dt * Elem<T>::load(u + row + b_col + n) : 0.f;
      cc[i] = n < ns ? Elem<T>::load(u + row + c_col + n) : 0.f;
      if (n == 0) aa[t] = expf(-rate * dt);
    }
    float xloc[TB][CS];
#pragma unroll
    for (int t = 0; t < TB; ++t) {
#pragma unroll
      for (int c = 0; c < CS; ++c)
        xloc[t][c] = (t < tb && owns && j0 + c < vdim) ? Elem<T>::load(u + (size_t)(t0 + t) * C + head * vdim + j0 + c) : 0.f;
    }
    __syncthreads();
    float outs[TB * CS];      // this thread's share of the round's outputs: [token][column]
#pragma unroll
    for (int i = 0; i < TB * CS; ++i) outs[i] = 0.f;
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb) {
        const float decay = aa[t];
        float o[CS] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r0 = 0; r0 < RS; r0 += 4) {
          const float4 b4 = *reinterpret_cast<const float4*>(bb + t * nsp + k0 + r0);
          const float4 c4 = *reinterpret_cast<const float4*>(cc + t * nsp + k0 + r0);
          const float bv[4] = {b4.x, b4.y, b4.z, b4.w}, cv[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int c = 0; c < CS; ++c) {
              s[r0 + e][c] = fmaf(decay, s[r0 + e][c], bv[e] * xloc[t][c]);
              if (MODE != 1) o[c] = fmaf(cv[e], s[r0 + e][c], o[c]);
            }
          }
        }
        if (MODE == 1) {
          decayed *= decay;
        } else {
#pragma unroll
          for (int c = 0; c < CS; ++c)      // (the skip term once a column group: in its first lane's share)
            outs[t * CS + c] = ks == 0 ? fmaf(d_skip, xloc[t][c], o[c]) : o[c];
        }
      }
    }
    if (MODE != 1) {
      // the sums over the KS lanes that share the column group (every lane of the wave takes part)
      static_assert(TB * CS == 32, "sum_and_deal takes 32 values");
      sum_and_deal<TB * CS, KS / 2>(outs, ks);
      constexpr int LEFT = KS <= TB * CS ? TB * CS / KS : 1;           // sums a lane is left with
      constexpr int SHARE = KS > TB * CS ? KS / (TB * CS) : 1;         // lanes that are left with the same sum
      const int base = ks * LEFT / SHARE;
      const bool writes = owns && (ks & (SHARE - 1)) == 0;
#pragma unroll
      for (int i = 0; i < LEFT; ++i) {
        const int t = (base + i) / CS, c = (base + i) % CS;
        if (writes && t < tb && j0 + c < vdim) y[(size_t)(t0 + t) * inner + head * vdim + j0 + c] = outs[i];
      }
    }
    __syncthreads();     // (the next round's staging writes what this round has read)
  }
  if (MODE != 2 && owns) {
#pragma unroll
    for (int r = 0; r < RS; ++r)      // (columns behind vdim stay zeros: their x is zero)
      if (k0 + r < ns) *reinterpret_cast<float4*>(S + r * 4) = make_float4(s[r][0], s[r][1], s[r][2], s[r][3]);
  }
  if (MODE == 1 && tid == 0 && blockIdx.z == 0) chunk_decay[place] = decayed;
}

// Per (request, head), a thread an element of the state: the chunks in order.  chunk_state holds every
// chunk's end state from zeros on entry and its start state on return; the request's state moves to the
// end of the step's tokens.
__global__ __launch_bounds__(256) void ssd_chunk_starts_kernel(
    float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
    float* __restrict__ chunk_state, const float* __restrict__ chunk_decay, int heads, int elems, int chunk) {
  const int req = blockIdx.x, head = blockIdx.y;
  const int count = (q_start[req + 1] - q_start[req] + chunk - 1) / chunk;
  int before = 0;
  for (int r = 0; r < req; ++r) before += (q_start[r + 1] - q_start[r] + chunk - 1) / chunk;
  float* S = state + ((size_t)state_slots[req] * heads + head) * elems;
  for (int e = blockIdx.z * blockDim.x + threadIdx.x; e < elems; e += gridDim.z * blockDim.x) {
    float s = S[e];
    for (int ci = 0; ci < count; ++ci) {
      const size_t place = (size_t)(before + ci) * heads + head;
      const float local = chunk_state[place * elems + e];
      chunk_state[place * elems + e] = s;
      s = fmaf(chunk_decay[place], s, local);
    }
    S[e] = s;
  }
}

// A wave a (token, part of the row): out = g / rms(g) * weight with g = y * silu(z).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    const float* __restrict__ y, SsmIn z_in, long ld, int z_col, const float* __restrict__ weight,
    T* __restrict__ out, long pairs, int inner, int groups, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const long pair = (long)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (pair >= pairs) return;
  const long n = pair / groups;
  const int g = (int)(pair - n * groups), size = inner / groups;
  const size_t at = (size_t)n * inner + (size_t)g * size;
  const size_t zat = (size_t)n * ld + z_col + (size_t)g * size;
  float ss = 0.f;
  for (int x = lane; x < size; x += kWave) {
    const float v = y[at + x] * silu(load_in<T>(z_in, zat + x));
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)size + eps);
  for (int x = lane; x < size; x += kWave) {
    const float v = y[at + x] * silu(load_in<T>(z_in, zat + x));
    Elem<T>::store(out + at + x, v * rstd * weight[(size_t)g * size + x]);
  }
}

// The same for long parts of the row: a block a (token, part), a thread up to kHold elements in registers
// (beyond that the products are formed again for the second pass).
constexpr int kHold = 8;
template <typename T>
__global__ __launch_bounds__(1024) void gated_group_norm_block_kernel(
    const float* __restrict__ y, SsmIn z_in, long ld, int z_col, const float* __restrict__ weight,
    T* __restrict__ out, int inner, int groups, float eps) {
  __shared__ float scratch[16];
  const long pair = blockIdx.x;
  const long n = pair / groups;
  const int g = (int)(pair - n * groups), size = inner / groups;
  const size_t at = (size_t)n * inner + (size_t)g * size;
  const size_t zat = (size_t)n * ld + z_col + (size_t)g * size;
  float held[kHold];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kHold; ++i) {
    const int x = threadIdx.x + i * blockDim.x;
    held[i] = x < size ? y[at + x] * silu(load_in<T>(z_in, zat + x)) : 0.f;
    ss = fmaf(held[i], held[i], ss);
  }
  for (int x = threadIdx.x + kHold * blockDim.x; x < size; x += blockDim.x) {
    const float v = y[at + x] * silu(load_in<T>(z_in, zat + x));
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)size + eps);
#pragma unroll
  for (int i = 0; i < kHold; ++i) {
    const int x = threadIdx.x + i * blockDim.x;
    if (x < size) Elem<T>::store(out + at + x, held[i] * rstd * weight[(size_t)g * size + x]);
  }
  for (int x = threadIdx.x + kHold * blockDim.x; x < size; x += blockDim.x) {
    const float v = y[at + x] * silu(load_in<T>(z_in, zat + x));
    Elem<T>::store(out + at + x, v * rstd * weight[(size_t)g * size + x]);
  }
}

template <typename T>
int launch_scan(const void* u, int C, SsmIn dt, long ld, int dt_col, const float* dt_bias, const float* a_log,
                const float* skip, float* state, const int* q_start, const int* state_slots, float* y, int R,
                int heads, int groups, int ns, int vdim, int splits, int chunk, int max_chunks, float* chunk_state,
                float* chunk_decay, hipStream_t stream) {
  ScanShape sh;
  sh.heads = heads;
  sh.groups = groups;
  sh.ns = ns;
  sh.vdim = vdim;
  // rows a thread (4, or more where the state is long) and threads a column group (a power of two up to a wave)
  const int rs = ns <= 256 ? 4 : ns <= 512 ? 8 : 16;
  const int ks = ns <= 16 ? 4 : ns <= 64 ? 16 : ns <= 128 ? 32 : 64;
  if (ns > 1024) return -1;
  sh.slices = ks;
  const int col_groups = (vdim + 3) / 4;
  sh.columns = max(1, min((col_groups + splits - 1) / splits, 1024 / ks));
  const int shares = (col_groups + sh.columns - 1) / sh.columns;
  const int threads = (sh.columns * ks + kWave - 1) / kWave * kWave;
  const size_t lds = ((size_t)2 * kScanTokens * ks * rs + kScanTokens) * 4;
  const dim3 grid(chunk > 0 ? R * max_chunks : R, heads, shares);
#define TK_SSD_AS(RS, KS, MODE)                                                                               \
  {                                                                                                           \
    if (lds > 48 * 1024) {                                                                                    \
      static bool raised = false;                                                                             \
      if (!raised) {                                                                                          \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&ssd_scan_kernel<T, RS, KS, MODE>),             \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024) != hipSuccess)         \
          return -1;                                                                                          \
        raised = true;                                                                                        \
      }                                                                                                       \
    }                                                                                                         \
    ssd_scan_kernel<T, RS, KS, MODE><<<grid, threads, lds, stream>>>((const T*)u, C, dt, ld, dt_col, dt_bias, \
                                                                    a_log, skip, state, q_start, state_slots, \
                                                                    y, sh, chunk, max_chunks, chunk_state,    \
                                                                    chunk_decay);                             \
  }
#define TK_SSD(MODE)                               \
  {                                                \
    if (rs == 16) TK_SSD_AS(16, 64, MODE)          \
    else if (rs == 8) TK_SSD_AS(8, 64, MODE)       \
    else if (ks == 64) TK_SSD_AS(4, 64, MODE)      \
    else if (ks == 32) TK_SSD_AS(4, 32, MODE)      \
    else if (ks == 16) TK_SSD_AS(4, 16, MODE)      \
    else TK_SSD_AS(4, 4, MODE)                     \
  }
  if (chunk <= 0) {
    TK_SSD(0)
    return launch_status();
  }
  TK_SSD(1)
  const int elems = (vdim + 3) / 4 * ns * 4;
  ssd_chunk_starts_kernel<<<dim3(R, heads, (elems + 1023) / 1024), 256, 0, stream>>>(state, q_start, state_slots, chunk_state,
                                                                                   chunk_decay, heads, elems, chunk);
  TK_SSD(2)
#undef TK_SSD
#undef TK_SSD_AS
  return launch_status();
}

}  // namespace

// proj: [N, ld] in dtype, or float32 (in_f32; possibly `parts` partial sums part_stride elements apart);
// the convolution's C channels start at column col0.  w float32 [C, taps], bias float32 [C], state float32
// [slots, taps - 1, C].  out: [N, C] in dtype.  max_tokens: the most tokens a request brings to the step.
TK_API int tk_conv_silu(int dtype, const void* proj, int in_f32, int parts, long part_stride, long ld, int col0,
                        const float* w, const float* bias, float* state, const int* q_start, const int* state_slots,
                        void* out, int R, int C, int taps, int max_tokens, hipStream_t stream) {
  if (R <= 0 || max_tokens <= 0) return 0;
  if (C < 1 || taps < 1 || taps > kMaxTaps || parts < 1 || (parts > 1 && !in_f32) || col0 < 0 || ld < col0 + C) return -1;
  const SsmIn in{proj, in_f32 || dtype == 0, parts, part_stride};
  const int segments = (max_tokens + kConvSegment - 1) / kConvSegment;
  const dim3 grid((C + 255) / 256, R, segments);
  if (grid.y > 65535 || grid.z > 65535) return -1;
  const int update = segments == 1 && taps > 1;
  if (dtype == 0)
    conv_silu_kernel<float><<<grid, 256, 0, stream>>>(in, ld, col0, w, bias, state, q_start, state_slots, (float*)out, C, taps, update);
  else
    conv_silu_kernel<bf16_t><<<grid, 256, 0, stream>>>(in, ld, col0, w, bias, state, q_start, state_slots, (bf16_t*)out, C, taps, update);
  if (!update && taps > 1) {
    const dim3 cgrid((C + 255) / 256, R);
    if (dtype == 0) conv_carry_kernel<float><<<cgrid, 256, 0, stream>>>(in, ld, col0, state, q_start, state_slots, C, taps);
    else conv_carry_kernel<bf16_t><<<cgrid, 256, 0, stream>>>(in, ld, col0, state, q_start, state_slots, C, taps);
  }
  return launch_status();
}

// u: [N, C] in dtype, C = heads * vdim + 2 * groups * ns ([x | B | C]).  dt: column dt_col .. + heads of rows
// ld long (dtype, float32 or partial sums).  state float32 [slots, heads, ceil(vdim / 4), ns, 4] (a head's columns
// in groups of four, the columns behind vdim zeros).  y float32 [N, heads * vdim].
// splits: blocks that share a head's value columns.  chunk > 0: portions are cut into chunks of so many tokens
// that run side by side; max_chunks: the most chunks a request of the step has; chunk_state float32
// [chunks of the step, heads, ceil(vdim / 4), ns, 4] and chunk_decay float32 [chunks of the step, heads] are scratch.
TK_API int tk_ssd_scan(int dtype, const void* u, const void* dt, int dt_f32, int dt_parts, long dt_stride, long ld,
                       int dt_col, const float* dt_bias, const float* a_log, const float* skip, float* state,
                       const int* q_start, const int* state_slots, float* y, int R, int heads, int groups, int ns,
                       int vdim, int splits, int chunk, int max_chunks, float* chunk_state, float* chunk_decay,
                       hipStream_t stream) {
  if (R <= 0) return 0;
  if (chunk < 0 || (chunk > 0 && (max_chunks < 1 || chunk_state == nullptr || chunk_decay == nullptr ||
                                  (long)R * max_chunks > 0x7fffffffL)))
    return -1;
  if (heads < 1 || groups < 1 || heads % groups != 0 || ns < 1 || vdim < 1 || vdim > 1024 || splits < 1 || R > 65535 ||
      heads > 65535 || dt_parts < 1 || (dt_parts > 1 && !dt_f32))
    return -1;
  const SsmIn in{dt, dt_f32 || dtype == 0, dt_parts, dt_stride};
  const int C = heads * vdim + 2 * groups * ns;
  if (dtype == 0)
    return launch_scan<float>(u, C, in, ld, dt_col, dt_bias, a_log, skip, state, q_start, state_slots, y, R, heads,
                              groups, ns, vdim, splits, chunk, max_chunks, chunk_state, chunk_decay, stream);
  return launch_scan<bf16_t>(u, C, in, ld, dt_col, dt_bias, a_log, skip, state, q_start, state_slots, y, R, heads,
                             groups, ns, vdim, splits, chunk, max_chunks, chunk_state, chunk_decay, stream);
}

// y float32 [N, inner]; z: column z_col .. + inner of rows ld long; weight float32 [inner]; out [N, inner] in dtype.
TK_API int tk_gated_group_norm(int dtype, const float* y, const void* z, int z_f32, int z_parts, long z_stride, long ld,
                               int z_col, const float* weight, void* out, int N, int inner, int groups, float eps,
                               hipStream_t stream) {
  if (N <= 0) return 0;
  if (inner < 1 || groups < 1 || inner % groups != 0 || z_parts < 1 || (z_parts > 1 && !z_f32)) return -1;
  const SsmIn in{z, z_f32 || dtype == 0, z_parts, z_stride};
  const long pairs = (long)N * groups;
  const int size = inner / groups;
  if (size > 256) {
    // a block a (token, part): enough threads that each holds a few elements
    int threads = 64;
    while (threads < 1024 && threads * 4 < size) threads *= 2;
    if (pairs > 0x7fffffffL) return -1;
    if (dtype == 0) gated_group_norm_block_kernel<float><<<(unsigned)pairs, threads, 0, stream>>>(y, in, ld, z_col, weight, (float*)out, inner, groups, eps);
    else gated_group_norm_block_kernel<bf16_t><<<(unsigned)pairs, threads, 0, stream>>>(y, in, ld, z_col, weight, (bf16_t*)out, inner, groups, eps);
    return launch_status();
  }
  const unsigned blocks = (unsigned)((pairs + 3) / 4);
  if (dtype == 0) gated_group_norm_kernel<float><<<blocks, 256, 0, stream>>>(y, in, ld, z_col, weight, (float*)out, pairs, inner, groups, eps);
  else gated_group_norm_kernel<bf16_t><<<blocks, 256, 0, stream>>>(y, in, ld, z_col, weight, (bf16_t*)out, pairs, inner, groups, eps);
  return launch_status();
}

TK_SLOTS(tk_conv_silu)
TK_SLOTS(tk_ssd_scan)
TK_SLOTS(tk_gated_group_norm)
