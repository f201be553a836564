// Paged attention of prompt portions on the matrix cores for the shapes the tuned kernels of
// attention_mfma.hip do not take: keys and values of unlike sizes (up to 512 channels each, keys in
// pieces of 8, values in blocks of 16), any number of query heads a kv head, a window or chunks, a sink.
// bf16 in, float32 softmax and accumulation.  Tokens that run alone have a form of their own (third
// kernel below) where a kv head has many query heads.
//
// A wave owns one tile (up to 16 consecutive tokens of one request) at one query head.  With fewer than
// four query heads a kv head, the four waves of a block take four heads of the same tile and every wave
// fetches its operands itself; with four and more, the waves of a block are heads of one kv head and
// share the operands through LDS (second kernel below).  Keys are walked 16 at a time, operands straight from the pages (no LDS):
//   S^T[key][token] = K[key][:] . Q[token][:]      v_mfma_f32_16x16x32_bf16, K rows as A (a lane
//       (key, kb) reads the 16-byte piece of dims 32 c + 8 kb of its key), Q rows as B, kept in registers
//   P^T = exp2(S^T * c - m[token])                  float32, a token's column per lane
//   O^T[dim][token] += V^T[dim][key] P^T[key][token] v_mfma_f32_16x16x16_bf16, V^T rows as A (a lane
//       (dim, kb) reads the 8 bytes of keys 4 kb .. 4 kb + 3 of its dim), P^T as B: the first product's
//       result layout is the second's B operand layout.
// What a token sees besides causality is given by `span`: 0 everything before it, W > 0 the last W
// positions, -C < 0 the positions of its own chunk of C; with a window, `keep` > 0 leaves the first
// `keep` positions of the sequence visible too (their stages of 16 keys are walked first, then the walk
// jumps to the window's first stage).  sinks: null, or float32 [nh]: exp(sinks[a])
// is one more term of head a's denominator.
//
// Cache pages: K [nkv][hd/8][ps][8], V [nkv][vd/16][ps/4][16][4]; ps a multiple of 16, so that 16
// consecutive keys from a multiple of 16 lie in one page.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

union Frag8 {
  uint4 u;
  bf16x8 v;
};
union Frag4 {
  uint2 u;
  short4v v;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr int kHeadsPerBlock = 4;

// KCH: 32-wide chunks of the key size the instance holds (hd <= 32 KCH); DBL: 16-wide blocks of the
// value size (vd <= 16 DBL).  Chunks and blocks behind the true sizes are skipped (the same for every lane).
template <int KCH, int DBL>
__global__ __launch_bounds__(kHeadsPerBlock * 64) void attention_tiles_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ tile_first, const int* __restrict__ tile_count,
    bf16_t* __restrict__ out, int nh, int nkv, int hd, int vd, int ps, float scale_log2, int span, int keep,
    const float* __restrict__ sinks) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, kb = lane >> 4;
  const int head = blockIdx.y * kHeadsPerBlock + wave;
  if (head >= nh) return;   // (the waves of a block never wait for one another)
  const int tile = blockIdx.x;
  const int n0 = tile_first[tile], cnt = tile_count[tile];
  const int kvh = head / (nh / nkv);
  const int pos0 = positions[n0];                 // the tile's tokens stand at pos0, pos0 + 1, ...
  const int my = min(col, cnt - 1);               // (columns behind the tile's last token repeat it and are not written)
  const int pos = pos0 + my;
  const int first = span > 0 ? max(pos - span + 1, 0) : span < 0 ? pos - pos % (-span) : 0;
  const int lo = span > 0 ? max(pos0 - span + 1, 0) : span < 0 ? pos0 - pos0 % (-span) : 0;   // the first token's first key
  const int hi = pos0 + cnt - 1;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t k_page = (size_t)nkv * hd * ps, v_page = (size_t)nkv * vd * ps;
  const size_t k_head = (size_t)kvh * hd * ps, v_head = (size_t)kvh * vd * ps;
  const int kch = (hd + 31) >> 5, dbl = vd >> 4;

  bf16x8 qreg[KCH];
  const bf16_t* qp = q + ((size_t)(n0 + my) * nh + head) * hd + kb * 8;
#pragma unroll
  for (int c = 0; c < KCH; ++c) {
    Frag8 f;
    f.u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(qp + c * 32) : make_uint4(0, 0, 0, 0);
    qreg[c] = f.v;
  }
  float m_run = -INFINITY, l_run = 0.f;
  float4v acc[DBL];
#pragma unroll
  for (int d = 0; d < DBL; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  const int c_first = lo & ~15;
  for (int c0 = keep > 0 ? 0 : c_first; c0 <= hi; c0 = (c0 + 16 >= keep && c0 + 16 < c_first) ? c_first : c0 + 16) {
    const int page = table[c0 / ps], off = c0 % ps;
    const bf16_t* kp = k_cache + (size_t)page * k_page + k_head + (size_t)(off + col) * 8;
    const bf16_t* vp = v_cache + (size_t)page * v_page + v_head + (size_t)((off >> 2) + kb) * 64 + col * 4;
    Frag8 kreg[KCH];
#pragma unroll
    for (int c = 0; c < KCH; ++c)
      kreg[c].u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(kp + (size_t)(c * 4 + kb) * ps * 8)
                                         : make_uint4(0, 0, 0, 0);
    Frag4 vreg[DBL];
#pragma unroll
    for (int d = 0; d < DBL; ++d)
      vreg[d].u = d < dbl ? *reinterpret_cast<const uint2*>(vp + (size_t)d * (ps >> 2) * 64) : make_uint2(0, 0);
    float4v sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KCH; ++c)
      if (c < kch) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[c].v, qreg[c], sc, 0, 0, 0);
    // this lane: keys c0 + 4 kb + e of token `col`
    float sv[4];
    bool seen[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = c0 + kb * 4 + e;
      seen[e] = (key >= first || key < keep) && key <= pos;
      sv[e] = seen[e] ? sc[e] * scale_log2 : -INFINITY;     // (a key that no token wrote may hold anything: chosen, not computed)
    }
    float tmax = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m_run, tmax);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;   // a token that has seen no key yet
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float pr[4], psum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      pr[e] = seen[e] ? fast_exp2(sv[e] - m_safe) : 0.f;
      psum += pr[e];
    }
    l_run = l_run * alpha + psum;
    Frag4 pb;
    pb.u = make_uint2(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]));
    const bool edge = c0 + 15 > hi;   // keys behind the tile's last token are not written yet
    const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
#pragma unroll
    for (int d = 0; d < DBL; ++d) {
      if (d >= dbl) continue;
      short4v tv = vreg[d].v;
      if (edge) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c0 + kb * 4 + e > hi) tv[e] = 0;
      }
      float4v a = acc[d];
      if (rescale) a *= alpha;
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tv, pb.v, a, 0, 0, 0);
    }
  }

  float l = l_run;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (sinks) l += fast_exp2(sinks[head] * 1.4426950408889634f - m_run);
  if (col >= cnt) return;
  const float inv = 1.f / l;
  // acc[d][e] = O^T[dim 16 d + 4 kb + e][token col]
  bf16_t* op = out + ((size_t)(n0 + col) * nh + head) * vd + kb * 4;
#pragma unroll
  for (int d = 0; d < DBL; ++d) {
    if (d >= dbl) continue;
    uint2 o;
    o.x = pack_bf16x2(acc[d][0] * inv, acc[d][1] * inv);
    o.y = pack_bf16x2(acc[d][2] * inv, acc[d][3] * inv);
    *reinterpret_cast<uint2*>(op + d * 16) = o;
  }
}

// The same products for kv heads with four query heads and more: a block of HB waves takes HB heads of
// ONE kv head at one tile and shares every 16 keys' operands through LDS (each wave of the kernel above
// fetches them from L2 for itself: with 32 heads on one kv head that is L2's rate, not the matrix
// cores').  A stage is the 16 keys' slice of the K page (hd/8 runs of 256 bytes) and of the V page
// (vd/16 runs of 512 bytes), copied as they lie, so the operand reads are those of the pages: a lane's
// 16-byte key piece at ((4 c + kb) 16 + key) 8, its 8-byte value piece at ((4 d + kb) 16 + dim) 4.  Two
// stages: the next one is fetched into registers before this one's products and written after them,
// one barrier a stage.  Operands are read from LDS per instruction, which leaves a wave under 256
// registers: two waves a SIMD.
template <int KCH, int DBL, int HB>
__global__ __launch_bounds__(HB * 64) void attention_tiles_shared_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ tile_first, const int* __restrict__ tile_count,
    bf16_t* __restrict__ out, int nh, int nkv, int hd, int vd, int ps, float scale_log2, int span, int keep,
    const float* __restrict__ sinks) {
  extern __shared__ __attribute__((aligned(16))) bf16_t stage_s[];   // two stages of (hd + vd) * 16 elements
  constexpr int THREADS = HB * 64;
  constexpr int KPT = (KCH * 64 + THREADS - 1) / THREADS;    // 16-byte pieces of K (hd / 8 * 16 = 2 hd) a thread copies
  constexpr int VPT = (DBL * 32 + THREADS - 1) / THREADS;    // and of V (vd / 16 * 32 = 2 vd)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, kb = lane >> 4;
  const int group = nh / nkv, blocks_per_kv = (group + HB - 1) / HB;
  const int kvh = blockIdx.y / blocks_per_kv;
  const int in_group = (blockIdx.y % blocks_per_kv) * HB + wave;
  const bool computes = in_group < group;                   // (a wave without a head still copies and waits)
  const int head = kvh * group + (computes ? in_group : 0);
  const int tile = blockIdx.x;
  const int n0 = tile_first[tile], cnt = tile_count[tile];
  const int pos0 = positions[n0];
  const int my = min(col, cnt - 1);
  const int pos = pos0 + my;
  const int first = span > 0 ? max(pos - span + 1, 0) : span < 0 ? pos - pos % (-span) : 0;
  const int lo = span > 0 ? max(pos0 - span + 1, 0) : span < 0 ? pos0 - pos0 % (-span) : 0;
  const int hi = pos0 + cnt - 1;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t k_page = (size_t)nkv * hd * ps, v_page = (size_t)nkv * vd * ps;
  const size_t k_head = (size_t)kvh * hd * ps, v_head = (size_t)kvh * vd * ps;
  const int kch = (hd + 31) >> 5, dbl = vd >> 4;
  const int k_pieces = 2 * hd, v_pieces = 2 * vd;           // 16-byte pieces of a stage
  const int stage_elems = (hd + vd) * 16;

  bf16x8 qreg[KCH];
  const bf16_t* qp = q + ((size_t)(n0 + my) * nh + head) * hd + kb * 8;
#pragma unroll
  for (int c = 0; c < KCH; ++c) {
    Frag8 f;
    f.u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(qp + c * 32) : make_uint4(0, 0, 0, 0);
    qreg[c] = f.v;
  }
  float m_run = -INFINITY, l_run = 0.f;
  float4v acc[DBL];
#pragma unroll
  for (int d = 0; d < DBL; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  uint4 kt[KPT], vt[VPT];
  // piece p of K: run j = p / 16 (8 dims), key p % 16; piece p of V: block d = p / 32, 16 bytes r = p % 32 of its 512
#define TK_SFETCH(C0_)                                                                                         \
  {                                                                                                            \
    const int page_ = table[(C0_) / ps], off_ = (C0_) % ps;                                                    \
    const bf16_t* kp_ = k_cache + (size_t)page_ * k_page + k_head + (size_t)off_ * 8;                          \
    const bf16_t* vp_ = v_cache + (size_t)page_ * v_page + v_head + (size_t)(off_ >> 2) * 64;                  \
    _Pragma("unroll") for (int i = 0; i < KPT; ++i) {                                                          \
      const int p_ = i * THREADS + threadIdx.x;                                                                \
      if (p_ < k_pieces) kt[i] = *reinterpret_cast<const uint4*>(kp_ + ((size_t)(p_ >> 4) * ps + (p_ & 15)) * 8); \
    }                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < VPT; ++i) {                                                          \
      const int p_ = i * THREADS + threadIdx.x;                                                                \
      if (p_ < v_pieces) vt[i] = *reinterpret_cast<const uint4*>(vp_ + (size_t)(p_ >> 5) * (ps >> 2) * 64 + (p_ & 31) * 8); \
    }                                                                                                          \
  }
#define TK_SSTORE(BUF_)                                                                                        \
  {                                                                                                            \
    bf16_t* ks_ = stage_s + (size_t)(BUF_) * stage_elems;                                                      \
    bf16_t* vs_ = ks_ + hd * 16;                                                                               \
    _Pragma("unroll") for (int i = 0; i < KPT; ++i) {                                                          \
      const int p_ = i * THREADS + threadIdx.x;                                                                \
      if (p_ < k_pieces) *reinterpret_cast<uint4*>(ks_ + (size_t)p_ * 8) = kt[i];                              \
    }                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < VPT; ++i) {                                                          \
      const int p_ = i * THREADS + threadIdx.x;                                                                \
      if (p_ < v_pieces) *reinterpret_cast<uint4*>(vs_ + (size_t)p_ * 8) = vt[i];                              \
    }                                                                                                          \
  }
  const int c_first = lo & ~15;
  const int c_start = keep > 0 ? 0 : c_first;
  TK_SFETCH(c_start)
  TK_SSTORE(0)
  __syncthreads();
  int buf = 0;
  for (int c0 = c_start, c_next; c0 <= hi; c0 = c_next, buf ^= 1) {
    c_next = (c0 + 16 >= keep && c0 + 16 < c_first) ? c_first : c0 + 16;    // (past the kept first positions: on to the window)
    const bool more = c_next <= hi;
    if (more) TK_SFETCH(c_next)
    if (computes) {
      const bf16_t* ks = stage_s + (size_t)buf * stage_elems;
      const bf16_t* vs = ks + hd * 16;
      float4v sc = {0.f, 0.f, 0.f, 0.f}, sc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KCH; c += 2) {
        if (c < kch) {     // (the same for every lane; a piece behind the key's end is absent from the stage: zeros)
          Frag8 kf;
          kf.u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(ks + ((size_t)(c * 4 + kb) * 16 + col) * 8)
                                        : make_uint4(0, 0, 0, 0);
          sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qreg[c], sc, 0, 0, 0);
        }
        if (c + 1 < kch) {
          Frag8 kf;
          kf.u = ((c + 1) * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(ks + ((size_t)((c + 1) * 4 + kb) * 16 + col) * 8)
                                              : make_uint4(0, 0, 0, 0);
          sc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qreg[c + 1], sc2, 0, 0, 0);
        }
      }
      sc += sc2;
      float sv[4];
      bool seen[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = c0 + kb * 4 + e;
        seen[e] = (key >= first || key < keep) && key <= pos;
        sv[e] = seen[e] ? sc[e] * scale_log2 : -INFINITY;
      }
      float tmax = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
      const float m_new = fmaxf(m_run, tmax);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2(m_run - m_safe);
      m_run = m_new;
      float pr[4], psum = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pr[e] = seen[e] ? fast_exp2(sv[e] - m_safe) : 0.f;
        psum += pr[e];
      }
      l_run = l_run * alpha + psum;
      Frag4 pb;
      pb.u = make_uint2(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]));
      const bool edge = c0 + 15 > hi;
      const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
#pragma unroll
      for (int d = 0; d < DBL; ++d) {
        if (d >= dbl) continue;
        Frag4 vf;
        vf.u = *reinterpret_cast<const uint2*>(vs + ((size_t)(d * 4 + kb) * 16 + col) * 4);
        short4v tv = vf.v;
        if (edge) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (c0 + kb * 4 + e > hi) tv[e] = 0;
        }
        float4v a = acc[d];
        if (rescale) a *= alpha;
        acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tv, pb.v, a, 0, 0, 0);
      }
    }
    if (more) TK_SSTORE(buf ^ 1)
    __syncthreads();
  }
#undef TK_SFETCH
#undef TK_SSTORE

  if (!computes) return;
  float l = l_run;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (sinks) l += fast_exp2(sinks[head] * 1.4426950408889634f - m_run);
  if (col >= cnt) return;
  const float inv = 1.f / l;
  bf16_t* op = out + ((size_t)(n0 + col) * nh + head) * vd + kb * 4;
#pragma unroll
  for (int d = 0; d < DBL; ++d) {
    if (d >= dbl) continue;
    uint2 o;
    o.x = pack_bf16x2(acc[d][0] * inv, acc[d][1] * inv);
    o.y = pack_bf16x2(acc[d][2] * inv, acc[d][3] * inv);
    *reinterpret_cast<uint2*>(op + d * 16) = o;
  }
}

template <int KCH, int DBL, int HB>
static int launch_shared(const void* q, const void* k_cache, const void* v_cache, const int* block_tables, int max_pages,
                         const int* positions, const int* req_of_token, const int* tile_first, const int* tile_count,
                         int num_tiles, void* out, int nh, int nkv, int hd, int vd, int ps, float scale, int span, int keep,
                         const float* sinks, hipStream_t stream) {
  const int group = nh / nkv;
  const size_t lds = (size_t)2 * (hd + vd) * 16 * sizeof(bf16_t);
  if (lds > 48 * 1024) {
    static bool raised = false;   // per template instance
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_tiles_shared_kernel<KCH, DBL, HB>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return -2;
      }
      raised = true;
    }
  }
  const dim3 grid(num_tiles, nkv * ((group + HB - 1) / HB));
  if (grid.y > 65535) return -1;
  attention_tiles_shared_kernel<KCH, DBL, HB><<<grid, HB * 64, lds, stream>>>(
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages, positions, req_of_token,
      tile_first, tile_count, (bf16_t*)out, nh, nkv, hd, vd, ps, scale * 1.4426950408889634f, span, keep, sinks);
  return launch_status();
}

// Tokens that run alone (decode) at kv heads with many query heads: the 16 columns of a wave's products
// are 16 HEADS of one kv head at one token, so a key or value fetched once serves them all.  The token's
// visible keys are walked 16 at a time; step t goes to wave t % (4 nsplit) of the token's nsplit blocks
// of four waves, operands straight from the pages.  Every wave leaves an unnormalised partial result
// (its maximum, its sum, its output) and a second kernel merges a head's partials in their order and
// adds the sink: no wave waits for another.
template <int KCH, int DBL>
__global__ __launch_bounds__(256) void attention_heads_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ single, float* __restrict__ part_o,
    float* __restrict__ part_ml, int nsplit, int nh, int nkv, int hd, int vd, int ps, float scale_log2, int span,
    int keep) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, kb = lane >> 4;
  const int group = nh / nkv, pieces = (group + 15) >> 4;
  const int kvh = blockIdx.y / pieces, in_group = (blockIdx.y % pieces) * 16 + col;
  const bool c_valid = in_group < group;
  const int head = kvh * group + min(in_group, group - 1);
  const int item = blockIdx.x, n0 = single[item];
  const int pos = positions[n0];
  const int first = span > 0 ? max(pos - span + 1, 0) : span < 0 ? pos - pos % (-span) : 0;
  const int* table = block_tables + (size_t)req_of_token[n0] * max_pages;
  const size_t k_page = (size_t)nkv * hd * ps, v_page = (size_t)nkv * vd * ps;
  const size_t k_head = (size_t)kvh * hd * ps, v_head = (size_t)kvh * vd * ps;
  const int kch = (hd + 31) >> 5, dbl = vd >> 4;
  const int parts = nsplit * 4, part = blockIdx.z * 4 + wave;

  bf16x8 qreg[KCH];
  const bf16_t* qp = q + ((size_t)n0 * nh + head) * hd + kb * 8;
#pragma unroll
  for (int c = 0; c < KCH; ++c) {
    Frag8 f;
    f.u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(qp + c * 32) : make_uint4(0, 0, 0, 0);
    qreg[c] = f.v;
  }
  float m_run = -INFINITY, l_run = 0.f;
  float4v acc[DBL];
#pragma unroll
  for (int d = 0; d < DBL; ++d) acc[d] = float4v{0.f, 0.f, 0.f, 0.f};

  // the stages of the walk in order: those of the kept first positions that lie before the window's first
  // stage, then the window's; stage s goes to part s % parts
  const int c_first = first & ~15;
  const int kept = min((keep + 15) >> 4, c_first >> 4);
  for (int st = part;; st += parts) {
    const int c0 = st < kept ? st * 16 : c_first + (st - kept) * 16;
    if (c0 > pos) break;
    const int page = table[c0 / ps], off = c0 % ps;
    const bf16_t* kp = k_cache + (size_t)page * k_page + k_head + (size_t)(off + col) * 8;
    const bf16_t* vp = v_cache + (size_t)page * v_page + v_head + (size_t)((off >> 2) + kb) * 64 + col * 4;
    Frag8 kreg[KCH];
#pragma unroll
    for (int c = 0; c < KCH; ++c)
      kreg[c].u = (c * 32 + kb * 8 < hd) ? *reinterpret_cast<const uint4*>(kp + (size_t)(c * 4 + kb) * ps * 8)
                                         : make_uint4(0, 0, 0, 0);
    Frag4 vreg[DBL];
#pragma unroll
    for (int d = 0; d < DBL; ++d)
      vreg[d].u = d < dbl ? *reinterpret_cast<const uint2*>(vp + (size_t)d * (ps >> 2) * 64) : make_uint2(0, 0);
    float4v sc = {0.f, 0.f, 0.f, 0.f}, sc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KCH; c += 2) {
      if (c < kch) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[c].v, qreg[c], sc, 0, 0, 0);
      if (c + 1 < kch) sc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[c + 1].v, qreg[c + 1], sc2, 0, 0, 0);
    }
    sc += sc2;
    float sv[4];
    bool seen[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = c0 + kb * 4 + e;
      seen[e] = (key >= first || key < keep) && key <= pos;
      sv[e] = seen[e] ? sc[e] * scale_log2 : -INFINITY;
    }
    float tmax = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, kWave));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, kWave));
    const float m_new = fmaxf(m_run, tmax);   // finite: a step holds at least one visible key
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    float pr[4], psum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      pr[e] = seen[e] ? fast_exp2(sv[e] - m_new) : 0.f;
      psum += pr[e];
    }
    l_run = l_run * alpha + psum;
    Frag4 pb;
    pb.u = make_uint2(pack_bf16x2(pr[0], pr[1]), pack_bf16x2(pr[2], pr[3]));
    const bool edge = c0 + 15 > pos;
#pragma unroll
    for (int d = 0; d < DBL; ++d) {
      if (d >= dbl) continue;
      short4v tv = vreg[d].v;
      if (edge) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c0 + kb * 4 + e > pos) tv[e] = 0;
      }
      float4v a = acc[d];
      a *= alpha;
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tv, pb.v, a, 0, 0, 0);
    }
  }
  float l = l_run;
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (!c_valid) return;
  // partial rows [item][head][part]: (maximum, sum), then the output
  const size_t prow = ((size_t)item * nh + head) * parts + part;
  if (kb == 0) {
    part_ml[prow * 2] = m_run;
    part_ml[prow * 2 + 1] = l;
  }
  float* po = part_o + prow * vd + kb * 4;
#pragma unroll
  for (int d = 0; d < DBL; ++d) {
    if (d >= dbl) continue;
    *reinterpret_cast<float4*>(po + d * 16) = make_float4(acc[d][0], acc[d][1], acc[d][2], acc[d][3]);
  }
}

// out[token][head] = sum_p w_p o_p / (sum_p w_p l_p + exp(sink)), w_p = exp2(m_p - max m); a part without
// keys has m = -inf and weighs nothing (its output is not read).  A block a (token, head): lane p of the
// first wave takes part p's maximum and sum (up to 64 parts), then a thread a value channel, the parts'
// outputs asked for eight at a time and added in their order.
__global__ __launch_bounds__(256) void attention_heads_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ single,
    bf16_t* __restrict__ out, int parts, int nh, int vd, const float* __restrict__ sinks) {
  __shared__ float w_s[64];
  __shared__ float inv_s;
  const int item = blockIdx.x, head = blockIdx.y;
  const size_t row = ((size_t)item * nh + head) * parts;
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    const float m = p < parts ? part_ml[(row + p) * 2] : -INFINITY;
    const float l = p < parts ? part_ml[(row + p) * 2 + 1] : 0.f;
    const float mx = wave_max(m);                       // finite: the part that holds the token's own key
    const float w = m == -INFINITY ? 0.f : fast_exp2(m - mx);
    float denom = wave_sum(w * (m == -INFINITY ? 0.f : l));
    if (sinks) denom += fast_exp2(sinks[head] * 1.4426950408889634f - mx);
    w_s[p] = w;
    if (p == 0) inv_s = 1.f / denom;
  }
  __syncthreads();
  const float inv = inv_s;
  bf16_t* op = out + ((size_t)single[item] * nh + head) * vd;
  const float* po = part_o + row * vd;
  for (int d = threadIdx.x; d < vd; d += blockDim.x) {
    float o = 0.f;
    for (int p0 = 0; p0 < parts; p0 += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = p0 + u;
        v[u] = (p < parts && w_s[p] != 0.f) ? po[(size_t)p * vd + d] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) o = fmaf(p0 + u < parts ? w_s[p0 + u] : 0.f, v[u], o);
    }
    op[d] = float_to_bf16(o * inv);
  }
}

}  // namespace

// Tiles of up to 16 consecutive tokens of one request (tile_first, tile_count), bfloat16.  Returns -2
// for a shape the kernel does not take (the caller uses the generic kernel).
TK_API int tk_attention_tiles(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                              int max_pages, const int* positions, const int* req_of_token, const int* tile_first,
                              const int* tile_count, int num_tiles, void* out, int nh, int nkv, int hd, int vd, int ps,
                              float scale, int span, int keep, const float* sinks, hipStream_t stream) {
  if (num_tiles <= 0) return 0;
  if (keep < 0 || (keep > 0 && span <= 0)) return -1;
  if (nkv <= 0 || nh % nkv != 0 || hd < 8 || hd % 8 != 0 || vd < 16 || vd % 16 != 0 || ps < 16 || ps % 16 != 0) return -2;
  if (hd > 512 || vd > 512 || (uintptr_t)q % 16 != 0 || (uintptr_t)k_cache % 16 != 0 || (uintptr_t)v_cache % 16 != 0 ||
      (uintptr_t)out % 8 != 0)
    return -2;
  const int group = nh / nkv;
  if (group >= 4) {
    // the heads of a kv head share its keys and values through LDS
#define TK_SHARED(KCH_, DBL_, HB_)                                                                              \
  launch_shared<KCH_, DBL_, HB_>(q, k_cache, v_cache, block_tables, max_pages, positions, req_of_token, tile_first, \
                                 tile_count, num_tiles, out, nh, nkv, hd, vd, ps, scale, span, keep, sinks, stream)
    if (hd <= 128 && vd <= 128) return group > 4 ? TK_SHARED(4, 8, 8) : TK_SHARED(4, 8, 4);
    if (hd <= 256 && vd <= 256) return group > 4 ? TK_SHARED(8, 16, 8) : TK_SHARED(8, 16, 4);
    return group > 4 ? TK_SHARED(16, 32, 8) : TK_SHARED(16, 32, 4);
#undef TK_SHARED
  }
  const dim3 grid(num_tiles, (nh + kHeadsPerBlock - 1) / kHeadsPerBlock);
  if (grid.y > 65535) return -1;
#define TK_TILES(KCH_, DBL_)                                                                                   \
  attention_tiles_kernel<KCH_, DBL_><<<grid, kHeadsPerBlock * 64, 0, stream>>>(                                \
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages, positions,    \
      req_of_token, tile_first, tile_count, (bf16_t*)out, nh, nkv, hd, vd, ps, scale * 1.4426950408889634f,    \
      span, keep, sinks)
  if (hd <= 128 && vd <= 128) TK_TILES(4, 8);
  else if (hd <= 256 && vd <= 256) TK_TILES(8, 16);
  else TK_TILES(16, 32);
#undef TK_TILES
  return launch_status();
}

// Single tokens (`single`: their rows, num_single of them), bfloat16, for kv heads with many query heads.
// part_o: float32 [num_single * nh * 4 nsplit * vd], part_ml: float32 [num_single * nh * 4 nsplit * 2].
TK_API int tk_attention_heads(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                              int max_pages, const int* positions, const int* req_of_token, const int* single,
                              int num_single, void* out, float* part_o, float* part_ml, int nsplit, int nh, int nkv,
                              int hd, int vd, int ps, float scale, int span, int keep, const float* sinks,
                              hipStream_t stream) {
  if (num_single <= 0) return 0;
  if (keep < 0 || (keep > 0 && span <= 0)) return -1;
  if (nkv <= 0 || nh % nkv != 0 || hd < 8 || hd % 8 != 0 || vd < 16 || vd % 16 != 0 || ps < 16 || ps % 16 != 0) return -2;
  if (hd > 512 || vd > 512 || (uintptr_t)q % 16 != 0 || (uintptr_t)k_cache % 16 != 0 || (uintptr_t)v_cache % 16 != 0 ||
      (uintptr_t)part_o % 16 != 0 || nsplit < 1 || nsplit > 16 || nh > 65535)    // (the merge: up to 64 parts)
    return -2;
  const int group = nh / nkv;
  const dim3 grid(num_single, nkv * ((group + 15) / 16), nsplit);
  if (grid.y > 65535) return -1;
#define TK_HEADS(KCH_, DBL_)                                                                                  \
  attention_heads_kernel<KCH_, DBL_><<<grid, 256, 0, stream>>>(                                               \
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages, positions,   \
      req_of_token, single, part_o, part_ml, nsplit, nh, nkv, hd, vd, ps, scale * 1.4426950408889634f, span, keep)
  if (hd <= 128 && vd <= 128) TK_HEADS(4, 8);
  else if (hd <= 256 && vd <= 256) TK_HEADS(8, 16);
  else TK_HEADS(16, 32);
#undef TK_HEADS
  attention_heads_merge_kernel<<<dim3(num_single, nh), vd <= 64 ? 64 : vd <= 128 ? 128 : 256, 0, stream>>>(  // (whole waves)
      part_o, part_ml, single, (bf16_t*)out, nsplit * 4, nh, vd, sinks);
  return launch_status();
}

TK_SLOTS(tk_attention_tiles)
TK_SLOTS(tk_attention_heads)
