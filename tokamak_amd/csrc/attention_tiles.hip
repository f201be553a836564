// Paged attention of prompt portions on the matrix cores for the shapes the tuned kernels of
// attention_mfma.hip do not take: keys and values of unlike sizes (up to 512 channels each, keys in
// pieces of 8, values in blocks of 16), any number of query heads a kv head, a window or chunks, a sink.
// bf16 in, float32 softmax and accumulation.
//
// A wave owns one tile (up to 16 consecutive tokens of one request) at one query head; the four
// waves of a block take four heads of the same tile, so what one asks of memory the others find in
// the CU's cache.  Keys are walked 16 at a time, operands straight from the pages (no LDS):
//   S^T[key][token] = K[key][:] . Q[token][:]      v_mfma_f32_16x16x32_bf16, K rows as A (a lane
//       (key, kb) reads the 16-byte piece of dims 32 c + 8 kb of its key), Q rows as B, kept in registers
//   P^T = exp2(S^T * c - m[token])                  float32, a token's column per lane
//   O^T[dim][token] += V^T[dim][key] P^T[key][token] v_mfma_f32_16x16x16_bf16, V^T rows as A (a lane
//       (dim, kb) reads the 8 bytes of keys 4 kb .. 4 kb + 3 of its dim), P^T as B: the first product's
//       result layout is the second's B operand layout.
// What a token sees besides causality is given by `span`: 0 everything before it, W > 0 the last W
// positions, -C < 0 the positions of its own chunk of C.  sinks: null, or float32 [nh]: exp(sinks[a])
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
    bf16_t* __restrict__ out, int nh, int nkv, int hd, int vd, int ps, float scale_log2, int span,
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

  for (int c0 = lo & ~15; c0 <= hi; c0 += 16) {
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
      seen[e] = key >= first && key <= pos;
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

}  // namespace

// Tiles of up to 16 consecutive tokens of one request (tile_first, tile_count), bfloat16.  Returns -2
// for a shape the kernel does not take (the caller uses the generic kernel).
TK_API int tk_attention_tiles(const void* q, const void* k_cache, const void* v_cache, const int* block_tables,
                              int max_pages, const int* positions, const int* req_of_token, const int* tile_first,
                              const int* tile_count, int num_tiles, void* out, int nh, int nkv, int hd, int vd, int ps,
                              float scale, int span, const float* sinks, hipStream_t stream) {
  if (num_tiles <= 0) return 0;
  if (nkv <= 0 || nh % nkv != 0 || hd < 8 || hd % 8 != 0 || vd < 16 || vd % 16 != 0 || ps < 16 || ps % 16 != 0) return -2;
  if (hd > 512 || vd > 512 || (uintptr_t)q % 16 != 0 || (uintptr_t)k_cache % 16 != 0 || (uintptr_t)v_cache % 16 != 0 ||
      (uintptr_t)out % 8 != 0)
    return -2;
  const dim3 grid(num_tiles, (nh + kHeadsPerBlock - 1) / kHeadsPerBlock);
  if (grid.y > 65535) return -1;
#define TK_TILES(KCH_, DBL_)                                                                                   \
  attention_tiles_kernel<KCH_, DBL_><<<grid, kHeadsPerBlock * 64, 0, stream>>>(                                \
      (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_pages, positions,    \
      req_of_token, tile_first, tile_count, (bf16_t*)out, nh, nkv, hd, vd, ps, scale * 1.4426950408889634f,    \
      span, sinks)
  if (hd <= 128 && vd <= 128) TK_TILES(4, 8);
  else if (hd <= 256 && vd <= 256) TK_TILES(8, 16);
  else TK_TILES(16, 32);
#undef TK_TILES
  return launch_status();
}

TK_SLOTS(tk_attention_tiles)
