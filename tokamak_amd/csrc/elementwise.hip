// Memory-bound kernels of one step: embedding gather, residual add + RMSNorm,
// rotary tables, per-head q/k norm + rotation + cache write, SiLU-gate product.
// The residual stream is float32 in both dtypes; norm statistics, rotation
// angles and the residual sum are float32.
#include "common.h"
#include "slots.h"

using namespace tk;

// ---------------------------------------------------------------------------
// embedding: resid[n, :] = float(table[ids[n], :]) * scale, or with `accumulate`
// resid[n, :] += float(table[ids[n], :]) * scale (the same rows added to the stream once
// more, for a model that feeds its input in again); an id outside [0, V) gives NaN
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ resid, int H, int V, float scale, int accumulate) {
  const int n = blockIdx.x;
  const int id = ids[n];
  float* out = resid + (size_t)n * H;
  if (id < 0 || id >= V) {
    for (int d = threadIdx.x; d < H; d += blockDim.x) out[d] = __uint_as_float(0x7fc00000u);
    return;
  }
  const T* row = table + (size_t)id * H;
  if (accumulate) {
    for (int d = threadIdx.x; d < H; d += blockDim.x) out[d] += Elem<T>::load(row + d) * scale;
  } else {
    for (int d = threadIdx.x; d < H; d += blockDim.x) out[d] = Elem<T>::load(row + d) * scale;
  }
}

TK_API int tk_embed_gather(int dtype, const void* table, const int* ids, float* resid, int N, int H,
                           int V, float scale, int accumulate, hipStream_t stream) {
  if (N <= 0) return 0;
  if (dtype == 0)
    embed_gather_kernel<float><<<N, 256, 0, stream>>>((const float*)table, ids, resid, H, V, scale, accumulate);
  else
    embed_gather_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)table, ids, resid, H, V, scale, accumulate);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Token ids that are still on the GPU: ids[slots[i]] = sampled[rows[i]].  A step may be
// launched before the host has read the tokens that the step before it sampled; its
// descriptor then names, for such a token, the row of the sampler's output to take it from.
// ---------------------------------------------------------------------------
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ sampled,
                                   const int* __restrict__ slots, const int* __restrict__ rows, int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) ids[slots[i]] = sampled[rows[i]];
}

TK_API int tk_feed_tokens(int* ids, const int* sampled, const int* slots, const int* rows, int count,
                          hipStream_t stream) {
  if (count <= 0) return 0;
  feed_tokens_kernel<<<(count + 255) / 256, 256, 0, stream>>>(ids, sampled, slots, rows, count);
  return launch_status();
}

// ---------------------------------------------------------------------------
// residual add + RMSNorm over rows of width H.
//   x = resid[row] (+ delta[row]);  if write_resid: resid[row] = x
//   out[m] = x * rsqrt(mean(x^2) + eps) * weight
// row = rows ? rows[m] : m.  With `rows`, write_resid must be 0 (a row could be
// named twice).
// ---------------------------------------------------------------------------
// delta may come as `parts` float32 partial sums, part_stride elements apart
// (a split-K product's output): they are added in order.
template <typename TD> struct Load4;
template <> struct Load4<float> {
  static __device__ __forceinline__ float4 at(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <> struct Load4<bf16_t> {
  static __device__ __forceinline__ float4 at(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
};
template <typename T> struct Store4;
template <> struct Store4<float> {
  static __device__ __forceinline__ void at(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Store4<bf16_t> {
  static __device__ __forceinline__ void at(bf16_t* p, float4 v) {
    uint2 u;
    u.x = pack_bf16x2(v.x, v.y);
    u.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

// Vector form: H a multiple of 4 and at most 4 * kNormGroups * blockDim.  A thread
// keeps its elements of the row in registers, and all loads of the partial sums
// are issued before the first add, so a row costs about one memory round trip.
constexpr int kNormGroups = 4;

template <typename T, typename TD>
__global__ __launch_bounds__(1024) void add_rmsnorm_vec_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, int parts, long part_stride,
    const int* __restrict__ rows, const float* __restrict__ weight, T* __restrict__ out, int H,
    float eps, int write_resid) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  const TD* dl = delta ? delta + row * H : nullptr;
  float4 xv[kNormGroups], wv[kNormGroups];
  float ss = 0.f;
  // the norm's weight is asked for with the stream, not after the rows' sums are known (a
  // memory round trip less in a kernel that is little else)
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    wv[g] = d < H ? *reinterpret_cast<const float4*>(weight + d) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    xv[g] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < H) {
      float4 v = *reinterpret_cast<const float4*>(x + d);
      if (dl) {
        int p = 0;
        for (; p + 8 <= parts; p += 8) {   // eight partial sums in flight, added in split order
          float4 q[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) q[u] = Load4<TD>::at(dl + (size_t)(p + u) * part_stride + d);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            v.x += q[u].x;
            v.y += q[u].y;
            v.z += q[u].z;
            v.w += q[u].w;
          }
        }
        for (; p + 4 <= parts; p += 4) {
          const float4 a = Load4<TD>::at(dl + (size_t)p * part_stride + d);
          const float4 b = Load4<TD>::at(dl + (size_t)(p + 1) * part_stride + d);
          const float4 c = Load4<TD>::at(dl + (size_t)(p + 2) * part_stride + d);
          const float4 e = Load4<TD>::at(dl + (size_t)(p + 3) * part_stride + d);
          v.x = (((v.x + a.x) + b.x) + c.x) + e.x;
          v.y = (((v.y + a.y) + b.y) + c.y) + e.y;
          v.z = (((v.z + a.z) + b.z) + c.z) + e.z;
          v.w = (((v.w + a.w) + b.w) + c.w) + e.w;
        }
        for (; p < parts; ++p) {
          const float4 a = Load4<TD>::at(dl + (size_t)p * part_stride + d);
          v.x += a.x;
          v.y += a.y;
          v.z += a.z;
          v.w += a.w;
        }
        if (write_resid) *reinterpret_cast<float4*>(x + d) = v;
      }
      xv[g] = v;
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    if (d < H) {
      const float4 w = wv[g];
      Store4<T>::at(o + d, make_float4(xv[g].x * rstd * w.x, xv[g].y * rstd * w.y,
                                       xv[g].z * rstd * w.z, xv[g].w * rstd * w.w));
    }
  }
}

template <typename T, typename TD>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TD* __restrict__ delta,
                                   int parts, long part_stride, const int* __restrict__ rows,
                                   const float* __restrict__ weight, T* __restrict__ out, int H,
                                   float eps, int write_resid) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  const TD* dl = delta ? delta + row * H : nullptr;
  float ss = 0.f;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (dl) {
      for (int p = 0; p < parts; ++p) v += Elem<TD>::load(dl + (size_t)p * part_stride + d);
      if (write_resid) x[d] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (dl && !write_resid)
      for (int p = 0; p < parts; ++p) v += Elem<TD>::load(dl + (size_t)p * part_stride + d);
    Elem<T>::store(o + d, v * rstd * weight[d]);
  }
}

// delta_f32: delta is float32 (possibly `parts` partial sums) whatever the dtype
TK_API int tk_add_rmsnorm(int dtype, float* resid, const void* delta, int delta_f32, int parts,
                          long part_stride, const int* rows, const float* weight, void* out, int M,
                          int H, float eps, int write_resid, hipStream_t stream) {
  if (M <= 0) return 0;
  if (rows && write_resid) return -1;
  if (parts < 1 || (parts > 1 && !delta_f32 && dtype != 0)) return -1;
  // vector form when the row fits a block's registers and everything is 16-byte aligned
  // one element group per thread when rows are few (short latency chain), four when many
  int threads = 64;
  while (threads < 1024 && threads * 4 * (M >= 512 ? kNormGroups : 1) < H) threads *= 2;
  const bool vec = H % 4 == 0 && H <= threads * 4 * kNormGroups && part_stride % 4 == 0 &&
                   ((uintptr_t)resid % 16 == 0) && ((uintptr_t)delta % 16 == 0) &&
                   ((uintptr_t)weight % 16 == 0) && ((uintptr_t)out % 16 == 0);
#define TK_NORM(KERNEL, T_, TD_)                                                                 \
  KERNEL<T_, TD_><<<M, threads, 0, stream>>>(resid, (const TD_*)delta, parts, part_stride, rows, \
                                             weight, (T_*)out, H, eps, write_resid)
  if (vec) {
    if (dtype == 0) TK_NORM(add_rmsnorm_vec_kernel, float, float);
    else if (delta_f32) TK_NORM(add_rmsnorm_vec_kernel, bf16_t, float);
    else TK_NORM(add_rmsnorm_vec_kernel, bf16_t, bf16_t);
  } else {
    threads = 256;
    if (dtype == 0) TK_NORM(add_rmsnorm_kernel, float, float);
    else if (delta_f32) TK_NORM(add_rmsnorm_kernel, bf16_t, float);
    else TK_NORM(add_rmsnorm_kernel, bf16_t, bf16_t);
  }
#undef TK_NORM
  return launch_status();
}

// ---------------------------------------------------------------------------
// rotary tables: angle = float(pos) * inv_freq[j]  (one float32 product, as the
// formula is written), cos/sin [N, half]
// ---------------------------------------------------------------------------
// `amplitude` multiplies both tables (1: as they are).
__global__ void rope_tables_kernel(const int* __restrict__ positions,
                                   const float* __restrict__ inv_freq, float* __restrict__ cos_t,
                                   float* __restrict__ sin_t, int N, int half, float amplitude) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * half) return;
  const int n = i / half, j = i - n * half;
  const float angle = __fmul_rn((float)positions[n], inv_freq[j]);
  const float c = cosf(angle), s = sinf(angle);
  cos_t[i] = amplitude == 1.f ? c : c * amplitude;
  sin_t[i] = amplitude == 1.f ? s : s * amplitude;
}

TK_API int tk_rope_tables(const int* positions, const float* inv_freq, float* cos_t, float* sin_t,
                          int N, int half, float amplitude, hipStream_t stream) {
  const int total = N * half;
  if (total <= 0) return 0;
  rope_tables_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, cos_t, sin_t, N,
                                                               half, amplitude);
  return launch_status();
}

// ---------------------------------------------------------------------------
// per-head RMSNorm of q and k, half-split rotation of the first `rot` dims,
// q written out, k and v written into the paged cache.
//
// qkv: [N, (nh + 2*nkv) * hd] (q heads, then k heads, then v heads); with
// nkv_in == 0 the input holds q heads only and nothing is stored.
// Cache pages (page_elems = nkv * hd * ps elements each):
//   K page: [nkv][hd/8][ps][8]   (8 consecutive dims of one token are adjacent,
//                                 then tokens, so lanes that hold consecutive
//                                 tokens read consecutive 16-byte pieces)
//   V page: [nkv][hd/16][ps/4][16][4]  (4 consecutive tokens of one dim adjacent,
//                                 then 16 dims, then groups of 4 tokens: the A
//                                 operand of the PV product, lane (dim, quad),
//                                 is 8 contiguous bytes and a wave reads 512
//                                 contiguous bytes)
// One wave per (token, head), four waves a block, each with an LDS row of its own.
// ---------------------------------------------------------------------------
constexpr int kMaxHeadDim = 512;
constexpr int kPairsPerBlock = 4;  // (token, head) pairs per block, one per wave

template <typename T, typename TIN>
__global__ void qknorm_rope_store_kernel(
    const TIN* __restrict__ qkv, int parts, long part_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ block_tables, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int nh, int nkv_in, int nkv, int hd, int rot, int ps, int max_pages,
    float eps, int num_pairs) {
  __shared__ float vecs[kPairsPerBlock][kMaxHeadDim];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int heads = nh + 2 * nkv_in;
  const int pair = blockIdx.x * kPairsPerBlock + wave;
  if (pair >= num_pairs) return;  // nothing below synchronises across waves
  const int n = pair / heads, head = pair - n * heads;
  float* vec = vecs[wave];
  const int row_width = heads * hd;
  const TIN* src = qkv + (size_t)n * row_width + (size_t)head * hd;
  const bool is_q = head < nh;
  const bool is_k = !is_q && head < nh + nkv_in;
  const float* w = is_q ? q_weight : (is_k ? k_weight : nullptr);

  float ss = 0.f;
  for (int d = lane; d < hd; d += kWave) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += Elem<TIN>::load(src + (size_t)p * part_stride + d);
    vec[d] = v;
    ss += v * v;
  }
  if (is_q || is_k) {
    if (w) {
      ss = wave_sum(ss);
      const float rstd = rsqrtf(ss / (float)hd + eps);
      wave_lds_sync();
      for (int d = lane; d < hd; d += kWave) vec[d] = vec[d] * rstd * w[d];
    }
    wave_lds_sync();
    // out[j] = x[j] cos_j - x[j+half] sin_j ; out[j+half] = x[j+half] cos_j + x[j] sin_j
    const int half = rot / 2;
    float lo[kMaxHeadDim / 2 / kWave], hi[kMaxHeadDim / 2 / kWave];
    int cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      const float c = cos_t[(size_t)n * half + j], s = sin_t[(size_t)n * half + j];
      const float a = vec[j], b = vec[j + half];
      lo[cnt] = a * c - b * s;
      hi[cnt] = b * c + a * s;
    }
    wave_lds_sync();
    cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      vec[j] = lo[cnt];
      vec[j + half] = hi[cnt];
    }
  }
  wave_lds_sync();

  if (is_q) {
    T* dst = q_out + ((size_t)n * nh + head) * hd;
    for (int d = lane; d < hd; d += kWave) Elem<T>::store(dst + d, vec[d]);
    return;
  }
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  const size_t page_elems = (size_t)nkv * hd * ps;
  if (is_k) {
    const int kvh = head - nh;
    T* base = k_cache + (size_t)page * page_elems + (size_t)kvh * hd * ps;
    for (int d = lane; d < hd; d += kWave)
      Elem<T>::store(base + ((size_t)(d >> 3) * ps + off) * 8 + (d & 7), vec[d]);
  } else {
    const int kvh = head - nh - nkv_in;
    T* base = v_cache + (size_t)page * page_elems + (size_t)kvh * hd * ps;
    for (int d = lane; d < hd; d += kWave)
      Elem<T>::store(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), vec[d]);
  }
}

// Fast form for head sizes 64 and 128 rotated over their full width (rot == HD):
// a lane owns 8 consecutive dims of one head (one 16-byte piece), so a wave covers
// 64*8/HD (token, head) pairs; the rotation partner (dim +- HD/2) sits HD/16 lanes away, the
// sum of squares is over HD/8 neighbouring lanes.  The query heads come token by token; the
// pairs behind them are the key heads and then the value heads, each head with its tokens in
// order, so that a wave holds consecutive tokens of one head and its cache writes fall next
// to each other in the page: a key piece (8 dims of one token) beside those of the next
// tokens, and the values of four tokens that fill one quad of a page (bfloat16: exchanged
// through LDS inside the wave) as the page's own 16-byte pieces of two dims by four keys,
// where token by token they are 2-byte stores 8 bytes apart.
template <typename T, typename TIN, int HD>
__global__ __launch_bounds__(256) void qknorm_rope_store_vec_kernel(
    const TIN* __restrict__ qkv, int parts, long part_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ block_tables,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int N, int nh, int nkv_in,
    int nkv, int ps, int max_pages, float eps, long num_pairs) {
  constexpr int LPH = HD / 8;  // lanes per head
  __shared__ uint4 s_quad[sizeof(T) == 2 ? 256 : 1];
  const long slot = ((long)blockIdx.x * blockDim.x + threadIdx.x) / LPH;  // (token, head) pair
  if (slot >= num_pairs) return;  // whole LPH-lane groups leave together
  const int sub = threadIdx.x % LPH, d0 = sub * 8;
  const int heads = nh + 2 * nkv_in;
  const long q_pairs = (long)N * nh;
  int n, head;
  if (slot < q_pairs) {
    n = (int)((unsigned)slot / (unsigned)nh);
    head = (int)((unsigned)slot - (unsigned)n * (unsigned)nh);
  } else {
    const unsigned behind = (unsigned)(slot - q_pairs), kv = behind / (unsigned)N;
    n = (int)(behind - kv * (unsigned)N);
    head = nh + (int)kv;
  }
  const bool is_q = head < nh, is_k = !is_q && head < nh + nkv_in;
  const TIN* src = qkv + (size_t)n * heads * HD + (size_t)head * HD + d0;
  float x[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = 0.f;
  for (int p = 0; p < parts; ++p) {
    const float4 a = Load4<TIN>::at(src + (size_t)p * part_stride);
    const float4 b = Load4<TIN>::at(src + (size_t)p * part_stride + 4);
    x[0] += a.x; x[1] += a.y; x[2] += a.z; x[3] += a.w;
    x[4] += b.x; x[5] += b.y; x[6] += b.z; x[7] += b.w;
  }
  if (is_q || is_k) {
    const float* w = is_q ? q_weight : k_weight;
    const int j0 = d0 % (HD / 2);  // index into the cos/sin row
    const float4 c0 = *reinterpret_cast<const float4*>(cos_t + (size_t)n * (HD / 2) + j0);
    const float4 c1 = *reinterpret_cast<const float4*>(cos_t + (size_t)n * (HD / 2) + j0 + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(sin_t + (size_t)n * (HD / 2) + j0);
    const float4 s1 = *reinterpret_cast<const float4*>(sin_t + (size_t)n * (HD / 2) + j0 + 4);
    const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
      for (int m = LPH / 2; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, kWave);
      const float rstd = rsqrtf(ss / (float)HD + eps);
      const float4 w0 = *reinterpret_cast<const float4*>(w + d0);
      const float4 w1 = *reinterpret_cast<const float4*>(w + d0 + 4);
      const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = x[e] * rstd * wv[e];
    }
    // first half: x cos - partner sin; second half: x cos + partner sin
    const float sign = (d0 < HD / 2) ? -1.f : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float partner = __shfl_xor(x[e], LPH / 2, kWave);
      x[e] = x[e] * cs[e] + sign * partner * sn[e];
    }
  }
  if (is_q) {
    Store4<T>::at(q_out + ((size_t)n * nh + head) * HD + d0, make_float4(x[0], x[1], x[2], x[3]));
    Store4<T>::at(q_out + ((size_t)n * nh + head) * HD + d0 + 4, make_float4(x[4], x[5], x[6], x[7]));
    return;
  }
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  const size_t page_elems = (size_t)nkv * HD * ps;
  if (is_k) {
    T* base = k_cache + (size_t)page * page_elems + (size_t)(head - nh) * HD * ps;
    T* dst = base + ((size_t)sub * ps + off) * 8;  // dims d0 .. d0+7 of this token: one 8-element piece
    Store4<T>::at(dst, make_float4(x[0], x[1], x[2], x[3]));
    Store4<T>::at(dst + 4, make_float4(x[4], x[5], x[6], x[7]));
  } else {
    T* base = v_cache + (size_t)page * page_elems + (size_t)(head - nh - nkv_in) * HD * ps;
    if constexpr (sizeof(T) == 2) {
      // Four pairs in a row (a "quad" of this wave) that are four consecutive tokens of one
      // request and head and fill one quad of keys in a page?
      constexpr int QL = 4 * LPH;  // lanes of a quad
      const int lane = threadIdx.x & 63, t = (lane / LPH) & 3;
      const int first = lane / QL * QL + sub;  // the lane with these dims in the quad's first pair
      const int req = req_of_token[n];
      const bool fits = n == __shfl(n, first, kWave) + t && pos == __shfl(pos, first, kWave) + t &&
                        req == __shfl(req, first, kWave) && head == __shfl(head, first, kWave) && ((pos - t) & 3) == 0;
      const unsigned long long all = QL == 64 ? ~0ull : ((1ull << (QL & 63)) - 1) << (lane / QL * QL);
      if ((__builtin_amdgcn_ballot_w64(fits) & all) == all) {
        // every lane leaves its four dim pairs; lane t of the quad takes pair t of all four tokens
        s_quad[threadIdx.x] = make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]),
                                         pack_bf16x2(x[6], x[7]));
        wave_lds_sync();
        const unsigned* words = reinterpret_cast<const unsigned*>(s_quad);
        const int quad0 = (int)threadIdx.x / QL * QL + sub;  // thread of the quad's first pair, these dims
        unsigned r[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = words[(quad0 + k * LPH) * 4 + t];  // token k: dims d, d + 1
        const int d = d0 + 2 * t;
        uint4 piece;  // [dim d: keys 0..3][dim d + 1: keys 0..3]
        piece.x = (r[0] & 0xffffu) | (r[1] << 16);
        piece.y = (r[2] & 0xffffu) | (r[3] << 16);
        piece.z = (r[0] >> 16) | (r[1] & 0xffff0000u);
        piece.w = (r[2] >> 16) | (r[3] & 0xffff0000u);
        *reinterpret_cast<uint4*>(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4) = piece;
        return;
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = d0 + e;
      Elem<T>::store(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), x[e]);
    }
  }
}

// in_f32: qkv is float32 (possibly `parts` partial sums, part_stride elements apart)
TK_API int tk_qknorm_rope_store(int dtype, const void* qkv, int in_f32, int parts, long part_stride,
                                const float* q_weight, const float* k_weight, const float* cos_t,
                                const float* sin_t, const int* positions, const int* req_of_token,
                                const int* block_tables, void* q_out, void* k_cache, void* v_cache,
                                int N, int nh, int nkv_in, int nkv, int hd, int rot, int ps,
                                int max_pages, float eps, hipStream_t stream) {
  if (N <= 0) return 0;
  if (hd > kMaxHeadDim || hd % 16 != 0 || ps % 4 != 0 || rot > hd || rot % 2 != 0) return -1;
  if (nkv_in != 0 && nkv_in != nkv) return -1;
  if (parts < 1 || (parts > 1 && !in_f32 && dtype != 0)) return -1;
  const long pairs = (long)N * (nh + 2 * nkv_in);
  if (pairs > 0x7fffffffL) return -1;
  if ((hd == 128 || hd == 64) && rot == hd && part_stride % 4 == 0 && (uintptr_t)qkv % 16 == 0 &&
      (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)cos_t % 16 == 0 &&
      (uintptr_t)sin_t % 16 == 0 && (!q_weight || (uintptr_t)q_weight % 16 == 0) &&
      (!k_weight || (uintptr_t)k_weight % 16 == 0) && (q_weight != nullptr) == (k_weight != nullptr)) {
    const long lanes = pairs * (hd / 8);
    const unsigned vgrid = (unsigned)((lanes + 255) / 256);
#define TK_QKV(T_, TIN_, HD_)                                                                     \
  qknorm_rope_store_vec_kernel<T_, TIN_, HD_><<<vgrid, 256, 0, stream>>>(                         \
      (const TIN_*)qkv, parts, part_stride, q_weight, k_weight, cos_t, sin_t, positions,          \
      req_of_token, block_tables, (T_*)q_out, (T_*)k_cache, (T_*)v_cache, N, nh, nkv_in, nkv, ps, \
      max_pages, eps, pairs)
    if (hd == 128) {
      if (dtype == 0) TK_QKV(float, float, 128);
      else if (in_f32) TK_QKV(bf16_t, float, 128);
      else TK_QKV(bf16_t, bf16_t, 128);
    } else {
      if (dtype == 0) TK_QKV(float, float, 64);
      else if (in_f32) TK_QKV(bf16_t, float, 64);
      else TK_QKV(bf16_t, bf16_t, 64);
    }
#undef TK_QKV
    return launch_status();
  }
  const unsigned grid = (unsigned)((pairs + kPairsPerBlock - 1) / kPairsPerBlock);
#define TK_QK(T_, TIN_)                                                                          \
  qknorm_rope_store_kernel<T_, TIN_><<<grid, kWave * kPairsPerBlock, 0, stream>>>(               \
      (const TIN_*)qkv, parts, part_stride, q_weight, k_weight, cos_t, sin_t, positions,         \
      req_of_token, block_tables, (T_*)q_out, (T_*)k_cache, (T_*)v_cache, nh, nkv_in, nkv, hd,   \
      rot, ps, max_pages, eps, (int)pairs)
  if (dtype == 0) TK_QK(float, float);
  else if (in_f32) TK_QK(bf16_t, float);
  else TK_QK(bf16_t, bf16_t);
#undef TK_QK
  return launch_status();
}

// ---------------------------------------------------------------------------
// out[n, i] = act(gu[n, i]) * gu[n, I + i]; act 0: silu(z) = z / (1 + exp(-z)), act 1: the tanh
// form of gelu, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------
__device__ __forceinline__ float gate_act(float z, int act) {
  if (act == 0) return z / (1.f + expf(-z));
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total, int act,
                                const float* __restrict__ bias) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / I;
  const int i = (int)(idx - n * I);
  float g = Elem<T>::load(gu + n * 2 * I + i);
  float u = Elem<T>::load(gu + n * 2 * I + I + i);
  if (bias) {     // (float32 [2 I]: the gate's biases, then the up projection's)
    g += bias[i];
    u += bias[I + i];
  }
  Elem<T>::store(out + idx, gate_act(g, act) * u);
}

// x[n, c] += bias[c] in place (float32 bias, the sum formed in float32)
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int H, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  Elem<T>::store(x + idx, Elem<T>::load(x + idx) + bias[idx % H]);
}

// 8 elements a thread (16-byte loads): I a multiple of 8, pointers 16-byte aligned
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                       int I, size_t total8, int act) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const int per_row = I / 8;
  const size_t n = idx / per_row;
  const int i = (int)(idx - n * per_row) * 8;
  const uint4 g = *reinterpret_cast<const uint4*>(gu + n * 2 * I + i);
  const uint4 u = *reinterpret_cast<const uint4*>(gu + n * 2 * I + I + i);
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  uint32_t ow[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
    ow[k] = pack_bf16x2(gate_act(g0, act) * u0, gate_act(g1, act) * u1);
  }
  *reinterpret_cast<uint4*>(out + n * I + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

TK_API int tk_add_bias(int dtype, void* x, const float* bias, int N, int H, hipStream_t stream) {
  if (N <= 0 || H <= 0) return 0;
  const size_t total = (size_t)N * H;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0) add_bias_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, bias, H, total);
  else add_bias_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, bias, H, total);
  return launch_status();
}

// bias: null, or float32 [2 I] added to the gate's and the up projection's halves before the activation
TK_API int tk_silu_mul(int dtype, const void* gu, void* out, int N, int I, int act, const float* bias,
                       hipStream_t stream) {
  if (N <= 0 || I <= 0) return 0;
  if (act != 0 && act != 1) return -1;
  const size_t total = (size_t)N * I;
  if (bias == nullptr && dtype == 1 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t total8 = total / 8;
    silu_mul_bf16x8_kernel<<<(unsigned)((total8 + 255) / 256), 256, 0, stream>>>(
        (const bf16_t*)gu, (bf16_t*)out, I, total8, act);
    return launch_status();
  }
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0)
    silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, I, total, act, bias);
  else
    silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total, act, bias);
  return launch_status();
}

// ---------------------------------------------------------------------------
// out[n, c] = scale[c] * (wa * a[n, c] + wb * b[n, c]), float32: the sum of a layer's parallel
// branches, each with its weight, times a per-coordinate layer scale.  a and b are each T,
// float32, or float32 partial sums of a split product; b may be absent.
template <typename T>
__device__ __forceinline__ float branch_value(const void* p, int f32, int parts, long part_stride, size_t idx) {
  if (!f32) return Elem<T>::load(reinterpret_cast<const T*>(p) + idx);
  const float* f = reinterpret_cast<const float*>(p);
  float s = f[idx];
  for (int i = 1; i < parts; ++i) s += f[idx + (size_t)i * part_stride];
  return s;
}

template <typename T>
__global__ void scaled_sum_kernel(const void* __restrict__ a, int a_f32, int a_parts, long a_stride, float wa,
                                  const void* __restrict__ b, int b_f32, int b_parts, long b_stride, float wb,
                                  const float* __restrict__ scale, float* __restrict__ out, int H, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float v = wa * branch_value<T>(a, a_f32, a_parts, a_stride, idx);
  if (b != nullptr) v = fmaf(wb, branch_value<T>(b, b_f32, b_parts, b_stride, idx), v);
  if (scale != nullptr) v *= scale[idx % H];
  out[idx] = v;
}

// four consecutive columns a thread: H a multiple of 4 (every row then starts on a border of four)
template <typename T>
__device__ __forceinline__ float4 branch_four(const void* p, int f32, int parts, long part_stride, size_t idx) {
  if (!f32) return Load4<T>::at(reinterpret_cast<const T*>(p) + idx);
  const float* f = reinterpret_cast<const float*>(p) + idx;
  float4 s = *reinterpret_cast<const float4*>(f);
  for (int i = 1; i < parts; ++i) {
    const float4 a = *reinterpret_cast<const float4*>(f + (size_t)i * part_stride);
    s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
  }
  return s;
}

template <typename T>
__global__ void scaled_sum_four_kernel(const void* __restrict__ a, int a_f32, int a_parts, long a_stride, float wa,
                                       const void* __restrict__ b, int b_f32, int b_parts, long b_stride, float wb,
                                       const float* __restrict__ scale, float* __restrict__ out, int H, size_t total4) {
  const size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i4 >= total4) return;
  const size_t idx = i4 * 4;
  const float4 x = branch_four<T>(a, a_f32, a_parts, a_stride, idx);
  float4 v = make_float4(wa * x.x, wa * x.y, wa * x.z, wa * x.w);
  if (b != nullptr) {
    const float4 y = branch_four<T>(b, b_f32, b_parts, b_stride, idx);
    v = make_float4(fmaf(wb, y.x, v.x), fmaf(wb, y.y, v.y), fmaf(wb, y.z, v.z), fmaf(wb, y.w, v.w));
  }
  if (scale != nullptr) {
    const float4 g = *reinterpret_cast<const float4*>(scale + idx % H);
    v = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
  }
  *reinterpret_cast<float4*>(out + idx) = v;
}

TK_API int tk_scaled_sum(int dtype, const void* a, int a_f32, int a_parts, long a_stride, float wa,
                         const void* b, int b_f32, int b_parts, long b_stride, float wb, const float* scale,
                         float* out, int N, int H, hipStream_t stream) {
  if (N <= 0 || H <= 0) return 0;
  const size_t total = (size_t)N * H;
  if (H % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0) {
    const size_t total4 = total / 4;
    const unsigned blocks4 = (unsigned)((total4 + 255) / 256);
    if (dtype == 0)
      scaled_sum_four_kernel<float><<<blocks4, 256, 0, stream>>>(a, a_f32, a_parts, a_stride, wa, b, b_f32, b_parts,
                                                                 b_stride, wb, scale, out, H, total4);
    else
      scaled_sum_four_kernel<bf16_t><<<blocks4, 256, 0, stream>>>(a, a_f32, a_parts, a_stride, wa, b, b_f32, b_parts,
                                                                  b_stride, wb, scale, out, H, total4);
    return launch_status();
  }
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0)
    scaled_sum_kernel<float><<<blocks, 256, 0, stream>>>(a, a_f32, a_parts, a_stride, wa, b, b_f32, b_parts,
                                                         b_stride, wb, scale, out, H, total);
  else
    scaled_sum_kernel<bf16_t><<<blocks, 256, 0, stream>>>(a, a_f32, a_parts, a_stride, wa, b, b_f32, b_parts,
                                                          b_stride, wb, scale, out, H, total);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Residual add of up to three parallel branches + norm over rows of width H.
//   x = resid[row] + scale * (a[row] + b[row] + c[row] + bias);  if write_resid: resid[row] = x
//   center: out[m] = (x - mean(x)) * rsqrt(mean((x - mean(x))^2) + eps) * weight   (a layer norm without a bias)
//   else:   out[m] = x * rsqrt(mean(x^2) + eps) * weight
// A branch is T, float32, or float32 partial sums (added in order); each may be absent, and so may
// the bias (float32 [H], one row for all).  The branches' sum is formed first, in float32, and
// added to the stream once.  weight2 / out2 (both or neither): the same normalised row times a
// second weight, for a layer whose two sub-layers each have a norm of their own over the same stream.
// ---------------------------------------------------------------------------
struct NormBranch {
  const void* p;
  int f32;
  int parts;
  long stride;
};

struct NormAdds {
  NormBranch a, b, c;
  const float* bias;
  float scale;
  __device__ __forceinline__ bool any() const { return a.p || b.p || c.p || bias; }
};

template <typename T>
__device__ __forceinline__ float4 branch_four(const NormBranch& b, size_t idx) {
  if (!b.f32) return Load4<T>::at(reinterpret_cast<const T*>(b.p) + idx);
  const float* f = reinterpret_cast<const float*>(b.p) + idx;
  float4 s = *reinterpret_cast<const float4*>(f);
  for (int i = 1; i < b.parts; ++i) {
    const float4 q = *reinterpret_cast<const float4*>(f + (size_t)i * b.stride);
    s.x += q.x; s.y += q.y; s.z += q.z; s.w += q.w;
  }
  return s;
}

// scale * (a + b + c + bias) at four consecutive columns from d of a row that starts at `at`
template <typename T>
__device__ __forceinline__ float4 adds_four(const NormAdds& n, size_t at, int d) {
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (n.a.p) s = branch_four<T>(n.a, at + d);
  if (n.b.p) {
    const float4 t = branch_four<T>(n.b, at + d);
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  if (n.c.p) {
    const float4 t = branch_four<T>(n.c, at + d);
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  if (n.bias) {
    const float4 t = *reinterpret_cast<const float4*>(n.bias + d);
    s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
  }
  if (n.scale != 1.f) { s.x *= n.scale; s.y *= n.scale; s.z *= n.scale; s.w *= n.scale; }
  return s;
}

template <typename T>
__device__ __forceinline__ float adds_value(const NormAdds& n, size_t at, int d) {
  float s = 0.f;
  if (n.a.p) s = branch_value<T>(n.a.p, n.a.f32, n.a.parts, n.a.stride, at + d);
  if (n.b.p) s += branch_value<T>(n.b.p, n.b.f32, n.b.parts, n.b.stride, at + d);
  if (n.c.p) s += branch_value<T>(n.c.p, n.c.f32, n.c.parts, n.c.stride, at + d);
  if (n.bias) s += n.bias[d];
  return n.scale != 1.f ? s * n.scale : s;
}

// Vector form: a thread keeps up to kNormGroups pieces of four elements of the row in registers.
template <typename T>
__global__ __launch_bounds__(1024) void add_norm2_vec_kernel(
    float* __restrict__ resid, NormAdds adds, const int* __restrict__ rows,
    const float* __restrict__ weight, T* __restrict__ out, const float* __restrict__ weight2, T* __restrict__ out2,
    int H, float eps, int write_resid, int center) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  float4 xv[kNormGroups], wv[kNormGroups];
  float sum = 0.f;
  const bool adding = adds.any();
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    wv[g] = d < H ? *reinterpret_cast<const float4*>(weight + d) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    xv[g] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < H) {
      float4 v = *reinterpret_cast<const float4*>(x + d);
      if (adding) {
        const float4 s = adds_four<T>(adds, row * H, d);
        v.x += s.x; v.y += s.y; v.z += s.z; v.w += s.w;
        if (write_resid) *reinterpret_cast<float4*>(x + d) = v;
      }
      xv[g] = v;
      sum += (v.x + v.y) + (v.z + v.w);
    }
  }
  float mean = 0.f;
  if (center) mean = block_sum(sum, scratch) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    if (d < H) {
      xv[g].x -= mean; xv[g].y -= mean; xv[g].z -= mean; xv[g].w -= mean;
      ss += xv[g].x * xv[g].x + xv[g].y * xv[g].y + xv[g].z * xv[g].z + xv[g].w * xv[g].w;
    }
  }
  ss = block_sum(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
#pragma unroll
  for (int g = 0; g < kNormGroups; ++g) {
    const int d = (g * blockDim.x + threadIdx.x) * 4;
    if (d < H) {
      const float4 w = wv[g];
      Store4<T>::at(o + d, make_float4(xv[g].x * rstd * w.x, xv[g].y * rstd * w.y,
                                       xv[g].z * rstd * w.z, xv[g].w * rstd * w.w));
      if (out2) {
        const float4 w2 = *reinterpret_cast<const float4*>(weight2 + d);
        Store4<T>::at(out2 + (size_t)m * H + d, make_float4(xv[g].x * rstd * w2.x, xv[g].y * rstd * w2.y,
                                                            xv[g].z * rstd * w2.z, xv[g].w * rstd * w2.w));
      }
    }
  }
}

// Any width and alignment: the row is walked three times (mean, variance, output).
template <typename T>
__global__ void add_norm2_kernel(float* __restrict__ resid, NormAdds adds,
                                 const int* __restrict__ rows, const float* __restrict__ weight,
                                 T* __restrict__ out, const float* __restrict__ weight2, T* __restrict__ out2,
                                 int H, float eps, int write_resid, int center) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t row = rows ? (size_t)rows[m] : (size_t)m;
  float* x = resid + row * H;
  const bool adding = adds.any();
  float sum = 0.f;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (adding) {
      v += adds_value<T>(adds, row * H, d);
      if (write_resid) x[d] = v;      // (the passes below then read the sum back)
    }
    sum += v;
  }
  const bool again = adding && !write_resid;    // the sum is not in the stream: it is formed again
  float mean = 0.f;
  if (center) mean = block_sum(sum, scratch) / (float)H;
  float ss = 0.f;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (again) v += adds_value<T>(adds, row * H, d);
    ss += (v - mean) * (v - mean);
  }
  ss = block_sum(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)H + eps);
  T* o = out + (size_t)m * H;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
    float v = x[d];
    if (again) v += adds_value<T>(adds, row * H, d);
    Elem<T>::store(o + d, (v - mean) * rstd * weight[d]);
    if (out2) Elem<T>::store(out2 + (size_t)m * H + d, (v - mean) * rstd * weight2[d]);
  }
}

TK_API int tk_add_norm2(int dtype, float* resid, const void* a, int a_f32, int a_parts, long a_stride,
                        const void* b, int b_f32, int b_parts, long b_stride, const void* c, int c_f32, int c_parts,
                        long c_stride, const float* bias, float scale, const int* rows,
                        const float* weight, void* out, const float* weight2, void* out2, int M, int H, float eps,
                        int write_resid, int center, hipStream_t stream) {
  if (M <= 0) return 0;
  if (rows && write_resid) return -1;
  if ((weight2 == nullptr) != (out2 == nullptr)) return -1;
  if (a_parts < 1 || b_parts < 1 || c_parts < 1 || (a_parts > 1 && !a_f32) || (b_parts > 1 && !b_f32) || (c_parts > 1 && !c_f32)) return -1;
  const NormAdds adds{{a, a_f32 || dtype == 0, a_parts, a_stride}, {b, b_f32 || dtype == 0, b_parts, b_stride},
                      {c, c_f32 || dtype == 0, c_parts, c_stride}, bias, scale};
  int threads = 64;
  while (threads < 1024 && threads * 4 * (M >= 512 ? kNormGroups : 1) < H) threads *= 2;
  const bool vec = H % 4 == 0 && H <= threads * 4 * kNormGroups && a_stride % 4 == 0 && b_stride % 4 == 0 && c_stride % 4 == 0 &&
                   ((uintptr_t)resid % 16 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0) &&
                   ((uintptr_t)c % 16 == 0) && ((uintptr_t)bias % 16 == 0) && ((uintptr_t)weight % 16 == 0) &&
                   ((uintptr_t)out % 16 == 0) && ((uintptr_t)weight2 % 16 == 0) && ((uintptr_t)out2 % 16 == 0);
  if (vec) {
    if (dtype == 0) add_norm2_vec_kernel<float><<<M, threads, 0, stream>>>(resid, adds, rows, weight, (float*)out, weight2, (float*)out2, H, eps, write_resid, center);
    else add_norm2_vec_kernel<bf16_t><<<M, threads, 0, stream>>>(resid, adds, rows, weight, (bf16_t*)out, weight2, (bf16_t*)out2, H, eps, write_resid, center);
  } else {
    if (dtype == 0) add_norm2_kernel<float><<<M, 256, 0, stream>>>(resid, adds, rows, weight, (float*)out, weight2, (float*)out2, H, eps, write_resid, center);
    else add_norm2_kernel<bf16_t><<<M, 256, 0, stream>>>(resid, adds, rows, weight, (bf16_t*)out, weight2, (bf16_t*)out2, H, eps, write_resid, center);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// ---------------------------------------------------------------------------
// Rotation of the first `rot` dims of q and k (half-split pairs, dim j with j + rot/2, or
// `interleaved` pairs, dim 2j with 2j + 1), THEN (unit) each head of q and k divided by
// its root mean square over all hd dims (times a weight per dim, if one is given), q written
// out, k and v written into the paged cache.  Keys and values may differ in size:
// qkv: [N, nh * hd + nkv_in * hd + nkv_in * vd] (q heads, k heads, v heads); with nkv_in == 0
// the input holds q heads only and nothing is stored.  Cache pages as above, the value page
// with a size of its own: K page [nkv][hdp/8][ps][8], V page [nkv][vdp/16][ps/4][16][4], where
// hdp >= hd and vdp >= vd are the sizes the pages and q_out are laid out for (hd rounded up to 8,
// vd to 16): the channels behind hd are written as zeros into q_out and never written in the
// pages (which start as zeros), so they add nothing to a score or an output.
// Values may be mixed with those another layer made for the same tokens (v_keep, float32
// [N, nkv * vd]): v_mode 1 leaves this layer's values there as they are projected; v_mode 2
// caches (1 - lambda) v + lambda v_keep with lambda = *v_lambda.
// One wave per (token, head), four waves a block, each with an LDS row of its own.
// ---------------------------------------------------------------------------
template <typename T, typename TIN>
__global__ void rope_norm_store_kernel(
    const TIN* __restrict__ qkv, int parts, long part_stride, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ block_tables, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, int nh, int nkv_in, int nkv, int hd, int vd, int hdp, int vdp, int rot, int ps,
    int max_pages, int unit, float eps, int num_pairs, int interleaved, float* __restrict__ v_keep, int v_mode,
    const float* __restrict__ v_lambda) {
  __shared__ float vecs[kPairsPerBlock][kMaxHeadDim];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int heads = nh + 2 * nkv_in;
  const int pair = blockIdx.x * kPairsPerBlock + wave;
  if (pair >= num_pairs) return;  // nothing below synchronises across waves
  const int n = pair / heads, head = pair - n * heads;
  float* vec = vecs[wave];
  const size_t row_width = (size_t)(nh + nkv_in) * hd + (size_t)nkv_in * vd;
  const bool is_q = head < nh;
  const bool is_k = !is_q && head < nh + nkv_in;
  const int width = (is_q || is_k) ? hd : vd;
  const size_t head_at = (is_q || is_k) ? (size_t)head * hd : (size_t)(nh + nkv_in) * hd + (size_t)(head - nh - nkv_in) * vd;
  const TIN* src = qkv + (size_t)n * row_width + head_at;
  for (int d = lane; d < width; d += kWave) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += Elem<TIN>::load(src + (size_t)p * part_stride + d);
    vec[d] = v;
  }
  wave_lds_sync();
  if (is_q || is_k) {
    const int half = rot / 2;
    float lo[kMaxHeadDim / 2 / kWave], hi[kMaxHeadDim / 2 / kWave];
    int cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      const float c = cos_t[(size_t)n * half + j], s = sin_t[(size_t)n * half + j];
      const float a = vec[interleaved ? 2 * j : j], b = vec[interleaved ? 2 * j + 1 : j + half];
      lo[cnt] = a * c - b * s;
      hi[cnt] = b * c + a * s;
    }
    wave_lds_sync();
    cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      vec[interleaved ? 2 * j : j] = lo[cnt];
      vec[interleaved ? 2 * j + 1 : j + half] = hi[cnt];
    }
    wave_lds_sync();
    if (unit) {
      float ss = 0.f;
      for (int d = lane; d < hd; d += kWave) ss += vec[d] * vec[d];
      ss = wave_sum(ss);
      const float rstd = 1.f / sqrtf(ss / (float)hd + eps);
      const float* w = is_q ? q_weight : k_weight;
      for (int d = lane; d < hd; d += kWave) vec[d] = vec[d] * rstd * (w ? w[d] : 1.f);   // (a lane rewrites what it read)
      wave_lds_sync();
    }
  }
  if (is_q) {
    T* dst = q_out + ((size_t)n * nh + head) * hdp;
    for (int d = lane; d < hdp; d += kWave) Elem<T>::store(dst + d, d < hd ? vec[d] : 0.f);
    return;
  }
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  if (is_k) {
    const int kvh = head - nh;
    T* base = k_cache + (size_t)page * ((size_t)nkv * hdp * ps) + (size_t)kvh * hdp * ps;
    for (int d = lane; d < hd; d += kWave)
      Elem<T>::store(base + ((size_t)(d >> 3) * ps + off) * 8 + (d & 7), vec[d]);
  } else {
    const int kvh = head - nh - nkv_in;
    T* base = v_cache + (size_t)page * ((size_t)nkv * vdp * ps) + (size_t)kvh * vdp * ps;
    float* keep = v_keep + ((size_t)n * nkv + kvh) * vd;
    const float lambda = v_mode == 2 ? *v_lambda : 0.f;
    for (int d = lane; d < vd; d += kWave) {
      float v = vec[d];
      if (v_mode == 1) keep[d] = v;
      else if (v_mode == 2) v = (1.f - lambda) * v + lambda * keep[d];
      Elem<T>::store(base + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), v);
    }
  }
}

// in_f32: qkv is float32 (possibly `parts` partial sums, part_stride elements apart)
TK_API int tk_rope_norm_store(int dtype, const void* qkv, int in_f32, int parts, long part_stride,
                              const float* q_weight, const float* k_weight, const float* cos_t,
                              const float* sin_t, const int* positions, const int* req_of_token,
                              const int* block_tables, void* q_out, void* k_cache, void* v_cache,
                              int N, int nh, int nkv_in, int nkv, int hd, int vd, int hdp, int vdp, int rot,
                              int ps, int max_pages, int unit, float eps, int interleaved, float* v_keep,
                              int v_mode, const float* v_lambda, hipStream_t stream) {
  if (N <= 0) return 0;
  if (hdp > kMaxHeadDim || vdp > kMaxHeadDim || hd < 1 || vd < 1 || hdp < hd || vdp < vd || hdp % 8 != 0 ||
      vdp % 16 != 0 || ps % 4 != 0 || rot > hd || rot % 2 != 0)
    return -1;
  if (v_mode < 0 || v_mode > 2 || (v_mode != 0 && v_keep == nullptr) || (v_mode == 2 && v_lambda == nullptr)) return -1;
  if (nkv_in != 0 && nkv_in != nkv) return -1;
  if (parts < 1 || (parts > 1 && !in_f32 && dtype != 0)) return -1;
  const long pairs = (long)N * (nh + 2 * nkv_in);
  if (pairs > 0x7fffffffL) return -1;
  const unsigned grid = (unsigned)((pairs + kPairsPerBlock - 1) / kPairsPerBlock);
#define TK_RN(T_, TIN_)                                                                          \
  rope_norm_store_kernel<T_, TIN_><<<grid, kWave * kPairsPerBlock, 0, stream>>>(                 \
      (const TIN_*)qkv, parts, part_stride, q_weight, k_weight, cos_t, sin_t, positions,         \
      req_of_token, block_tables, (T_*)q_out, (T_*)k_cache, (T_*)v_cache, nh, nkv_in, nkv, hd,   \
      vd, hdp, vdp, rot, ps, max_pages, unit, eps, (int)pairs, interleaved, v_keep, v_mode, v_lambda)
  if (dtype == 0) TK_RN(float, float);
  else if (in_f32) TK_RN(bf16_t, float);
  else TK_RN(bf16_t, bf16_t);
#undef TK_RN
  return launch_status();
}

// ---------------------------------------------------------------------------
// logits in place: x <- x * scale, then (cap > 0) x <- cap * tanh(x / cap)
// ---------------------------------------------------------------------------
__global__ void scale_softcap_kernel(float* __restrict__ x, size_t total, float scale, float cap) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float v = x[idx] * scale;
  if (cap > 0.f) v = cap * tanhf(v / cap);
  x[idx] = v;
}

TK_API int tk_scale_softcap(float* x, long total, float scale, float cap, hipStream_t stream) {
  if (total <= 0) return 0;
  scale_softcap_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(x, (size_t)total, scale, cap);
  return launch_status();
}

// the same entry points in slot form (slots.h), for launch lists
TK_SLOTS(tk_add_rmsnorm)
TK_SLOTS(tk_add_norm2)
TK_SLOTS(tk_rope_tables)
TK_SLOTS(tk_qknorm_rope_store)
TK_SLOTS(tk_silu_mul)
TK_SLOTS(tk_add_bias)
TK_SLOTS(tk_scaled_sum)
TK_SLOTS(tk_rope_norm_store)
TK_SLOTS(tk_scale_softcap)
