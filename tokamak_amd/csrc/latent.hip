// Kernels of attention over a cached latent: every token caches one normed latent c [rank] and one
// rotated key part [rot_dim] for all heads; a head's key is [W_uk c, rotated part] and its value
// W_uv c.  Here the keys' and values' up-projections are never formed for cached tokens: since
// (W_uk c) . q = c . (W_uk^T q), the query is carried into the latent's space once per token and
// head, the attention runs with ONE key/value head whose key is [c, rotated part] and whose value
// is c, and the head's output a (a weighted sum of latents) goes through W_uv afterwards.
//
//   latent_prepare: from the token's projections [q heads | latent | rotated key part]:
//     q head a = [dim unrotated | rot_dim rotated]: the unrotated part to q_plain [N, nh, dim], the
//     rotated part (first `rot` dims rotated, interleaved or half-split pairs) into
//     q_full[n, a, rank .. rank + rot_dim); channels behind up to the padded key size are zeros;
//     with q_weight (float32 [dim]) the unrotated part of every q unit is first divided by its root
//     mean square (eps) and multiplied by q_weight (a query that is itself a normed latent: one unit
//     of `dim` = its rank); q_full may then be absent;
//     c = latent / sqrt(mean(latent^2) + eps) * weight (float32 statistics), the key part rotated;
//     K page [1][hdp/8][ps][8] receives [c | rotated part], V page [1][vdp/16][ps/4][16][4] receives c.
//   head_linear: out[n, a, m] = sum_k x[n, a, k] W[a, m, k], a product per head, with row and head
//     strides on both sides (q_plain -> q_full[.., :rank] with W = W_uk^T per head; the attention's
//     output -> values with W = W_uv per head).  float32 accumulation over k ascending; bfloat16
//     operands whose rows fill 16-byte pieces run on the matrix cores.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

constexpr int kMaxUnit = 1024;     // elements of a q head or of latent + rotated part
constexpr int kUnitsPerBlock = 4;  // (token, unit) pairs a block, one per wave

template <typename T, typename TIN>
__global__ void latent_prepare_kernel(
    const TIN* __restrict__ proj, int parts, long part_stride, const float* __restrict__ c_weight,
    const float* __restrict__ q_weight, const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ block_tables, T* __restrict__ q_plain,
    T* __restrict__ q_full, T* __restrict__ k_cache, T* __restrict__ v_cache, int nh, int dim, int rot_dim,
    int rank, int hdp, int vdp, int rot, int interleaved, int ps, int max_pages, float eps, int stores,
    long num_units) {
  __shared__ float vecs[kUnitsPerBlock][kMaxUnit];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const long unit = (long)blockIdx.x * kUnitsPerBlock + wave;
  if (unit >= num_units) return;   // nothing below synchronises across waves
  const int units = nh + (stores ? 1 : 0);
  const int n = (int)(unit / units), a = (int)(unit - (long)n * units);
  const bool is_q = a < nh;
  const int qw = dim + rot_dim;
  const size_t row_width = (size_t)nh * qw + (stores ? rank + rot_dim : 0);
  const int width = is_q ? qw : rank + rot_dim;
  const int plain = is_q ? dim : rank;      // elements before the rotated part
  const TIN* src = proj + (size_t)n * row_width + (is_q ? (size_t)a * qw : (size_t)nh * qw);
  float* vec = vecs[wave];
  // four elements a lane at a time, each summed over the parts in order: their loads are all in flight
  for (int d0 = lane; d0 < width; d0 += 4 * kWave) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int p = 0; p < parts; ++p) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int d = min(d0 + u * kWave, width - 1);      // (past the end: the last element again, not kept)
        v[u] += Elem<TIN>::load(src + (size_t)p * part_stride + d);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (d0 + u * kWave < width) vec[d0 + u * kWave] = v[u];
  }
  wave_lds_sync();
  // rotation of the first `rot` dims of the rotated part
  {
    const int half = rot / 2;
    float* r = vec + plain;
    float lo[kMaxUnit / 2 / kWave], hi[kMaxUnit / 2 / kWave];
    int cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      const float c = cos_t[(size_t)n * half + j], s = sin_t[(size_t)n * half + j];
      const float u = r[interleaved ? 2 * j : j], v = r[interleaved ? 2 * j + 1 : j + half];
      lo[cnt] = u * c - v * s;
      hi[cnt] = v * c + u * s;
    }
    wave_lds_sync();
    cnt = 0;
    for (int j = lane; j < half; j += kWave, ++cnt) {
      r[interleaved ? 2 * j : j] = lo[cnt];
      r[interleaved ? 2 * j + 1 : j + half] = hi[cnt];
    }
    wave_lds_sync();
  }
  if (is_q) {
    T* qp = q_plain + ((size_t)n * nh + a) * dim;
    if (q_weight != nullptr) {
      float qs = 0.f;
      for (int d = lane; d < dim; d += kWave) qs += vec[d] * vec[d];
      qs = wave_sum(qs);
      const float q_rstd = 1.f / sqrtf(qs / (float)dim + eps);
      for (int d = lane; d < dim; d += kWave) Elem<T>::store(qp + d, vec[d] * q_rstd * q_weight[d]);
    } else {
      for (int d = lane; d < dim; d += kWave) Elem<T>::store(qp + d, vec[d]);
    }
    if (q_full == nullptr) return;
    T* qf = q_full + ((size_t)n * nh + a) * hdp;
    for (int d = rank + lane; d < hdp; d += kWave) Elem<T>::store(qf + d, d < rank + rot_dim ? vec[dim + d - rank] : 0.f);
    return;
  }
  float ss = 0.f;
  for (int d = lane; d < rank; d += kWave) ss += vec[d] * vec[d];
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)rank + eps);
  for (int d = lane; d < rank; d += kWave) vec[d] = vec[d] * rstd * c_weight[d];   // (a lane rewrites what it read)
  wave_lds_sync();
  const int pos = positions[n];
  const int page = block_tables[(size_t)req_of_token[n] * max_pages + pos / ps];
  const int off = pos % ps;
  T* kb = k_cache + (size_t)page * ((size_t)hdp * ps);
  for (int d = lane; d < rank + rot_dim; d += kWave)
    Elem<T>::store(kb + ((size_t)(d >> 3) * ps + off) * 8 + (d & 7), vec[d]);
  T* vb = v_cache + (size_t)page * ((size_t)vdp * ps);
  for (int d = lane; d < rank; d += kWave)
    Elem<T>::store(vb + ((size_t)(d >> 4) * (ps >> 2) + (off >> 2)) * 64 + (d & 15) * 4 + (off & 3), vec[d]);
}

// A block: 16 rows x 64 columns of one head; 256 threads, a thread 4 rows of one column.
constexpr int kHlRows = 16, kHlCols = 64, kHlK = 32;

template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(
    const T* __restrict__ x, long x_row, long x_head, const T* __restrict__ w, T* __restrict__ out,
    long out_row, long out_head, int N, int M, int K) {
  __shared__ float xs[kHlRows][kHlK];
  __shared__ float ws[kHlCols][kHlK + 1];
  const int head = blockIdx.z;
  const int n0 = blockIdx.y * kHlRows, m0 = blockIdx.x * kHlCols;
  const int col = threadIdx.x % kHlCols, rg = threadIdx.x / kHlCols;
  const T* wh = w + (size_t)head * M * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kHlK) {
    __syncthreads();
    for (int i = threadIdx.x; i < kHlRows * kHlK; i += 256) {
      const int r = i / kHlK, k = i - r * kHlK;
      xs[r][k] = (n0 + r < N && k0 + k < K) ? Elem<T>::load(x + (size_t)(n0 + r) * x_row + (size_t)head * x_head + k0 + k) : 0.f;
    }
    for (int i = threadIdx.x; i < kHlCols * kHlK; i += 256) {
      const int c = i / kHlK, k = i - c * kHlK;
      ws[c][k] = (m0 + c < M && k0 + k < K) ? Elem<T>::load(wh + (size_t)(m0 + c) * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kHlK; ++k) {
      const float wv = ws[col][k];
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = fmaf(xs[rg * 4 + r][k], wv, acc[r]);
    }
  }
  if (m0 + col < M) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int n = n0 + rg * 4 + r;
      if (n < N) Elem<T>::store(out + (size_t)n * out_row + (size_t)head * out_head + m0 + col, acc[r]);
    }
  }
}

// bfloat16 on the matrix cores: a wave owns 16 output columns of one head for NT tiles of 16 tokens;
// D^T[column][token] = W[column][:] . x[token][:] with v_mfma_f32_16x16x32_bf16, W rows as the A operand
// (lane (row, kb) holds k = 32 c + 8 kb .. + 8) and x rows as B, both as 16-byte pieces straight from
// memory (K a multiple of 8, rows 16-byte aligned); a lane ends with four consecutive columns of one
// token.  float32 accumulation over k ascending in chunks of 32.
typedef __bf16 hl_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hl_float4 __attribute__((ext_vector_type(4)));
union HlFrag {
  uint4 u;
  hl_bf16x8 v;
};

template <int NT>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(
    const bf16_t* __restrict__ x, long x_row, long x_head, const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
    long out_row, long out_head, int N, int M, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, kb = lane >> 4;
  const int head = blockIdx.z;
  const int m0 = (blockIdx.x * 4 + wave) * 16;
  const int n0 = blockIdx.y * 16 * NT;
  if (m0 >= M) return;   // (no barrier below)
  const int wrow = min(m0 + col, M - 1);
  const bf16_t* wp = w + ((size_t)head * M + wrow) * K + kb * 8;
  const bf16_t* xp[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
    xp[t] = x + (size_t)min(n0 + t * 16 + col, N - 1) * x_row + (size_t)head * x_head + kb * 8;
  hl_float4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = hl_float4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool there = k0 + kb * 8 < K;   // (K is a multiple of 8: a piece is whole or absent)
    HlFrag a, b[NT];
    a.u = there ? *reinterpret_cast<const uint4*>(wp + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < NT; ++t) b[t].u = there ? *reinterpret_cast<const uint4*>(xp[t] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[t].v, acc[t], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = n0 + t * 16 + col;
    if (n >= N) continue;
    bf16_t* op = out + (size_t)n * out_row + (size_t)head * out_head + m0 + kb * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (m0 + kb * 4 + e < M) op[e] = float_to_bf16(acc[t][e]);
  }
}

}  // namespace

// proj: [N, nh (dim + rot_dim) (+ rank + rot_dim if stores)] in dtype, or float32 (in_f32; possibly `parts`
// partial sums, part_stride elements apart).
TK_API int tk_latent_prepare(int dtype, const void* proj, int in_f32, int parts, long part_stride,
                             const float* c_weight, const float* q_weight, const float* cos_t, const float* sin_t,
                             const int* positions,
                             const int* req_of_token, const int* block_tables, void* q_plain, void* q_full,
                             void* k_cache, void* v_cache, int N, int nh, int dim, int rot_dim, int rank, int hdp,
                             int vdp, int rot, int interleaved, int ps, int max_pages, float eps, int stores,
                             hipStream_t stream) {
  if (N <= 0) return 0;
  if (nh < 1 || dim < 1 || rot_dim < 0 || rank < 1 || dim + rot_dim > kMaxUnit || rank + rot_dim > kMaxUnit ||
      hdp < rank + rot_dim || hdp % 8 != 0 || vdp < rank || vdp % 16 != 0 || rot % 2 != 0 || rot > rot_dim || ps % 4 != 0)
    return -1;
  if (parts < 1 || (parts > 1 && !in_f32 && dtype != 0)) return -1;
  if (rot > 0 && (cos_t == nullptr || sin_t == nullptr)) return -1;
  if (stores && (c_weight == nullptr || k_cache == nullptr || v_cache == nullptr)) return -1;
  if (q_plain == nullptr || (q_full == nullptr && (q_weight == nullptr || rot_dim != 0))) return -1;
  const long units = (long)N * (nh + (stores ? 1 : 0));
  if (units > 0x7fffffffL) return -1;
  const unsigned grid = (unsigned)((units + kUnitsPerBlock - 1) / kUnitsPerBlock);
#define TK_LP(T_, TIN_)                                                                                   \
  latent_prepare_kernel<T_, TIN_><<<grid, kWave * kUnitsPerBlock, 0, stream>>>(                           \
      (const TIN_*)proj, parts, part_stride, c_weight, q_weight, cos_t, sin_t, positions, req_of_token, block_tables, \
      (T_*)q_plain, (T_*)q_full, (T_*)k_cache, (T_*)v_cache, nh, dim, rot_dim, rank, hdp, vdp, rot,       \
      interleaved, ps, max_pages, eps, stores, units)
  if (dtype == 0) TK_LP(float, float);
  else if (in_f32) TK_LP(bf16_t, float);
  else TK_LP(bf16_t, bf16_t);
#undef TK_LP
  return launch_status();
}

// x [N][heads][K] with strides x_row, x_head (elements); w [heads][M][K]; out [N][heads][M] with strides.
TK_API int tk_head_linear(int dtype, const void* x, long x_row, long x_head, const void* w, void* out,
                          long out_row, long out_head, int N, int heads, int M, int K, hipStream_t stream) {
  if (N <= 0) return 0;
  if (heads < 1 || heads > 65535 || M < 1 || K < 1) return -1;
  if (dtype != 0 && K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0) {
    // (tokens in tiles of 16: four tiles a wave once there are enough of them to fill the GPU without)
    const int nt = (long)((N + 63) / 64) * ((M + 63) / 64) * heads >= 512 ? 4 : 1;
    const dim3 mgrid((M + 63) / 64, (N + 16 * nt - 1) / (16 * nt), heads);
    if (mgrid.y > 65535) return -1;
    if (nt == 4)
      head_linear_mfma_kernel<4><<<mgrid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w,
                                                             (bf16_t*)out, out_row, out_head, N, M, K);
    else
      head_linear_mfma_kernel<1><<<mgrid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w,
                                                             (bf16_t*)out, out_row, out_head, N, M, K);
    return launch_status();
  }
  const dim3 grid((M + kHlCols - 1) / kHlCols, (N + kHlRows - 1) / kHlRows, heads);
  if (grid.y > 65535) return -1;
  if (dtype == 0)
    head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_row, x_head, (const float*)w, (float*)out,
                                                        out_row, out_head, N, M, K);
  else
    head_linear_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)w,
                                                         (bf16_t*)out, out_row, out_head, N, M, K);
  return launch_status();
}

TK_SLOTS(tk_latent_prepare)
TK_SLOTS(tk_head_linear)
