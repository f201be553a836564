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

struct ScanShape {
  int heads, groups, ns, vdim;      // ns: the state's size per value channel
  int columns, slices, slice;       // threads = columns * slices; a thread owns `slice` state rows of a value column
};

// A block a (request, head, share of the value columns).  u: the convolution's output [N, C] = [x | B | C].
// dt_in: rows ld long, the heads' step sizes from column dt_col.  y: float32 [N, heads * vdim].
//
// Long portions are cut into chunks of `chunk` tokens that run side by side (the decay is one number a
// head and token, so a chunk's effect on the state is S_end = P S_start + L with P the product of its
// decays and L its end state from zeros):
//   MODE 1: a block a (request, chunk, head, share): from zeros to L and P, no output;
//   ssd_chunk_starts_kernel: per request the chunks in order, S_start of each, the request's new state;
//   MODE 2: the same blocks again, each from its S_start, with the outputs.
// MODE 0 walks a request's tokens in one block from the request's state.  A chunk's place in the scratch
// arrays is its number among all chunks of the step (requests in order).
template <typename T, int SLICE, int MODE>
__global__ __launch_bounds__(1024) void ssd_scan_kernel(
    const T* __restrict__ u, int C, SsmIn dt_in, long ld, int dt_col, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ skip, float* __restrict__ state,
    const int* __restrict__ q_start, const int* __restrict__ state_slots, float* __restrict__ y, ScanShape sh,
    int chunk, int max_chunks, float* __restrict__ chunk_state, float* __restrict__ chunk_decay) {
  constexpr int TB = kScanTokens;
  extern __shared__ float lds[];
  const int ns = sh.ns, vdim = sh.vdim, CT = sh.columns, KS = sh.slices, slice = sh.slice;
  const int nsp = (ns + 3) & ~3;
  float* bb = lds;                   // [TB][nsp]: dt B
  float* cc = bb + TB * nsp;         // [TB][nsp]: C
  float* aa = cc + TB * nsp;         // [TB]: the decay
  float* part = aa + TB;             // [KS][TB][CT]
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
  const int ks = tid / CT, jl = tid - ks * CT;
  const int j = blockIdx.z * CT + jl;
  const bool worker = ks < KS;
  const bool live = worker && j < vdim;
  const int k0 = ks * slice;
  const int kn = max(0, min(slice, ns - k0));
  const int inner = sh.heads * vdim;
  const int group = head / (sh.heads / sh.groups);
  const int b_col = inner + group * ns, c_col = inner + sh.groups * ns + group * ns;
  float* S = MODE == 0 ? state + ((size_t)state_slots[req] * sh.heads + head) * ns * vdim
                       : chunk_state + place * ns * vdim;
  float s[SLICE];
#pragma unroll
  for (int x = 0; x < SLICE; ++x) s[x] = (MODE != 1 && live && x < kn) ? S[(size_t)(k0 + x) * vdim + j] : 0.f;
  const float rate = expf(a_log[head]), bias = dt_bias[head], d_skip = skip[head];
  float decayed = 1.f;      // the product of the chunk's decays (MODE 1)

  for (int t0 = first; t0 < end; t0 += TB) {
    const int tb = min(TB, end - t0);
    for (int i = tid; i < tb * ns; i += nthreads) {
      const int t = i / ns, n = i - t * ns;
      const size_t row = (size_t)(t0 + t) * C;
      // (every element forms its token's step size itself: the same float32 operations, one barrier less)
      const float dt = softplus(load_in<T>(dt_in, (size_t)(t0 + t) * ld + dt_col + head) + bias);
      bb[t * nsp + n] = dt * Elem<T>::load(u + row + b_col + n);
      cc[t * nsp + n] = Elem<T>::load(u + row + c_col + n);
      if (n == 0) aa[t] = expf(-rate * dt);
    }
    float xloc[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t) xloc[t] = (t < tb && live) ? Elem<T>::load(u + (size_t)(t0 + t) * C + head * vdim + j) : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb) {
        const float xj = xloc[t], decay = aa[t];
        float o = 0.f;
#pragma unroll
        for (int x = 0; x < SLICE; x += 4) {
          if (x < kn) {
            const int at = t * nsp + k0 + x;        // (k0 and nsp are multiples of four)
            const float4 b4 = *reinterpret_cast<const float4*>(bb + at);
            const float4 c4 = *reinterpret_cast<const float4*>(cc + at);
            const float bv[4] = {b4.x, b4.y, b4.z, b4.w}, cv[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (x + e < kn) {
                s[x + e] = fmaf(decay, s[x + e], bv[e] * xj);
                if (MODE != 1) o = fmaf(cv[e], s[x + e], o);
              }
            }
          }
        }
        if (MODE == 1) decayed *= decay;
        else if (worker) part[(ks * TB + t) * CT + jl] = o;
      }
    }
    __syncthreads();
    if (MODE == 1) continue;     // (every thread alike; the barrier above keeps the staging of the next round off this one's reads)
    for (int t = worker ? ks : tb; t < tb; t += KS) {
      float o = 0.f;
      for (int q = 0; q < KS; ++q) o += part[(q * TB + t) * CT + jl];
      if (live) {
        const size_t at = (size_t)(t0 + t) * inner + head * vdim + j;
        y[at] = fmaf(d_skip, Elem<T>::load(u + (size_t)(t0 + t) * C + head * vdim + j), o);
      }
    }
    __syncthreads();     // (the next round's staging writes what this round's sums have read)
  }
  if (MODE != 2 && live) {
#pragma unroll
    for (int x = 0; x < SLICE; ++x)
      if (x < kn) S[(size_t)(k0 + x) * vdim + j] = s[x];
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
  sh.columns = splits > 1 ? (vdim + splits - 1) / splits : vdim;
  const int most = max(1, min(16, 1024 / sh.columns));
  sh.slice = max(4, ((ns + most - 1) / most + 3) / 4 * 4);
  sh.slices = (ns + sh.slice - 1) / sh.slice;
  if (sh.slice > 64) return -1;
  const int threads = (sh.columns * sh.slices + kWave - 1) / kWave * kWave;
  if (threads > 1024) return -1;
  const int nsp = (ns + 3) & ~3;
  const size_t lds = ((size_t)2 * kScanTokens * nsp + kScanTokens + (size_t)sh.slices * kScanTokens * sh.columns) * 4;
  if (lds > 64 * 1024) return -1;
  const dim3 grid(chunk > 0 ? R * max_chunks : R, heads, splits);
#define TK_SSD_AS(SLICE, MODE)                                                                                \
  ssd_scan_kernel<T, SLICE, MODE><<<grid, threads, lds, stream>>>((const T*)u, C, dt, ld, dt_col, dt_bias,    \
                                                                 a_log, skip, state, q_start, state_slots, y, \
                                                                 sh, chunk, max_chunks, chunk_state, chunk_decay)
#define TK_SSD(MODE)                     \
  {                                      \
    if (sh.slice <= 4) TK_SSD_AS(4, MODE);        \
    else if (sh.slice <= 16) TK_SSD_AS(16, MODE); \
    else TK_SSD_AS(64, MODE);                     \
  }
  if (chunk <= 0) {
    TK_SSD(0)
    return launch_status();
  }
  TK_SSD(1)
  const int elems = ns * vdim;
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
// ld long (dtype, float32 or partial sums).  state float32 [slots, heads, ns, vdim].  y float32 [N, heads * vdim].
// splits: blocks that share a head's value columns.  chunk > 0: portions are cut into chunks of so many tokens
// that run side by side; max_chunks: the most chunks a request of the step has; chunk_state float32
// [chunks of the step, heads, ns, vdim] and chunk_decay float32 [chunks of the step, heads] are scratch.
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
