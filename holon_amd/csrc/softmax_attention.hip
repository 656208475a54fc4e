// Softmax attention over a paged cache whose keys and values may differ in width, with an optional sliding window and an
// optional sink (a number per head that stands in the denominator and has no key or value). The general kernel: any
// element type, any sizes.
//
// A page of one site holds P tokens: keys [Hkv, P, D] (a token's key is a row), then values [Hkv, V, P] (transposed
// inside the page). One block of four waves per (token, head). Keys are walked in tiles of 64 that start at multiples
// of 64 (so a tile is whole pages wherever P divides 64), wave w taking tiles w, w + 4, ... of those the query sees; a
// lane takes one key of a tile: its score over D, with the query in LDS. For the values the lanes turn to the value
// columns: column d of a page is P neighbouring values, which a lane reads as 16-byte vectors and weighs with the
// tile's weights, handed round from the lanes that hold them. Every wave keeps a running maximum, sum and weighted
// values; the four are combined at the end in wave order, the sink joining there. Which keys a wave takes and in which
// order is decided by the query's position alone. Scores, weights and sums are float32.
#include "common.h"
#include "holon_hip.h"

#define SMX_MAX_D 512

namespace {

template <typename T, bool PAGED_VEC>
__global__ void __launch_bounds__(256) softmax_attention_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ pages, const int32_t* __restrict__ table,
    int table_stride, int table_rows, const int32_t* __restrict__ slots, const int32_t* __restrict__ token_row,
    const int32_t* __restrict__ positions, int heads, int kv_heads, int dim, int vdim, int page_size, int num_pages,
    const float* __restrict__ sink, float scale, int window, int key_vec) {
  __shared__ float q_s[SMX_MAX_D];
  __shared__ float sum_s[4][SMX_MAX_D];
  __shared__ float ml_s[4][2];
  const int w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x, h = blockIdx.y;
  const int pos = positions[t];
  const int hk = h / (heads / kv_heads);
  int slot = slots[token_row[t]];
  slot = slot < 0 ? 0 : (slot >= table_rows ? table_rows - 1 : slot);
  const int32_t* trow = table + (int64_t)slot * table_stride;
  const int64_t page_len = (int64_t)kv_heads * page_size * (dim + vdim);
  const int64_t val_base = (int64_t)kv_heads * page_size * dim + (int64_t)hk * vdim * page_size;
  const T* qp = q + ((int64_t)t * heads + h) * dim;
  for (int d = threadIdx.x; d < dim; d += 256) q_s[d] = Elem<T>::load(qp[d]);
  __syncthreads();
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[SMX_MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < SMX_MAX_D / WAVE; ++i) acc[i] = 0.f;
  constexpr int VEC = Elem<T>::kVec;     // key_vec: every key row starts on a 16-byte border and is whole vectors

  for (int j0 = (first / WAVE + w) * WAVE; j0 <= pos; j0 += 4 * WAVE) {
    const int key = j0 + lane;
    const bool seen = key >= first && key <= pos;
    float s = -INFINITY;
    int page = -1;
    if (seen && key / page_size < table_stride) {
      page = trow[key / page_size];
      if (page < 0 || page >= num_pages) page = -1;      // a table that does not hold the key: the key is not seen
    }
    if (page >= 0) {
      const int off = key % page_size;
      const T* kp = pages + page * page_len + ((int64_t)hk * page_size + off) * dim;
      float dot = 0.f;
      if (key_vec) {
        for (int d = 0; d < dim; d += VEC) {
          const uint4 raw = *reinterpret_cast<const uint4*>(kp + d);
          const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
          for (int i = 0; i < VEC; ++i) dot += q_s[d + i] * Elem<T>::load(e[i]);
        }
      } else {
        for (int d = 0; d < dim; ++d) dot += q_s[d] * Elem<T>::load(kp[d]);
      }
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    if (m_new == -INFINITY) continue;                    // nothing seen in this tile (the same in every lane)
    const float alpha = expf(m - m_new);                 // m = -inf before the first key: 0
    const float p = page >= 0 ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < SMX_MAX_D / WAVE; ++i) acc[i] *= alpha;
    if (PAGED_VEC) {
      // the tile is 64 / P whole pages; a lane reads its columns' P values of a page as vectors
      const int per = WAVE / page_size;
      for (int g = 0; g < per; ++g) {
        const int k0 = g * page_size;                    // the page's first key among the tile's
        if (j0 + k0 > pos || j0 + k0 + page_size <= first) continue;
        const int pg = __builtin_amdgcn_readlane(page, k0 + (j0 + k0 < first ? first - j0 - k0 : 0));
        if (pg < 0) continue;
        const T* vp = pages + pg * page_len + val_base;
#pragma unroll
        for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
          const int d = lane + i * WAVE;
          if (d >= vdim) break;
          const T* col = vp + (int64_t)d * page_size;
          float a = acc[i];
          for (int o = 0; o < page_size; o += VEC) {
            const uint4 raw = *reinterpret_cast<const uint4*>(col + o);
            const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
              const float pj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), k0 + o + u));
              a += pj * Elem<T>::load(e[u]);
            }
          }
          acc[i] = a;
        }
      }
    } else {
      const int count = min(WAVE, pos - j0 + 1);
      for (int j = 0; j < count; ++j) {                  // j is the same in every lane
        const int pg = __builtin_amdgcn_readlane(page, j);
        if (pg < 0) continue;
        const float pj = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), j));
        const T* vp = pages + pg * page_len + val_base + (j0 + j) % page_size;
#pragma unroll
        for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
          const int d = lane + i * WAVE;
          if (d < vdim) acc[i] += pj * Elem<T>::load(vp[(int64_t)d * page_size]);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < SMX_MAX_D / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < vdim) sum_s[w][d] = acc[i];
  }
  if (lane == 0) { ml_s[w][0] = m; ml_s[w][1] = l; }
  __syncthreads();
  float top = sink ? sink[h] : -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) top = fmaxf(top, ml_s[i][0]);
  float f[4], den = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[i] = ml_s[i][0] == -INFINITY ? 0.f : expf(ml_s[i][0] - top);
    den += ml_s[i][1] * f[i];
  }
  if (sink) den += expf(sink[h] - top);
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  for (int d = threadIdx.x; d < vdim; d += 256) {
    const float o = ((sum_s[0][d] * f[0] + sum_s[1][d] * f[1]) + sum_s[2][d] * f[2]) + sum_s[3][d] * f[3];
    out[((int64_t)t * heads + h) * vdim + d] = Elem<T>::store(o * inv);
  }
}
}  // namespace

extern "C" int holon_softmax_attention(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, int table_rows, const int32_t* slots,
                                       const int32_t* token_row, const int32_t* positions, int tokens, int heads,
                                       int kv_heads, int dim, int vdim, int page_size, int num_pages, const float* sink,
                                       float scale, int window, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "softmax_attention: %d/%d heads", heads,
              kv_heads);
  HOLON_CHECK(dim > 0 && dim <= SMX_MAX_D && vdim > 0 && vdim <= SMX_MAX_D,
              "softmax_attention: head sizes %d/%d (at most %d)", dim, vdim, SMX_MAX_D);
  HOLON_CHECK(page_size > 0 && num_pages > 0 && window >= 0 && table_stride > 0 && table_rows > 0,
              "softmax_attention: bad page geometry");
  if (tokens == 0) return 0;
  HOLON_CHECK(heads <= 65535, "softmax_attention: %d heads exceed one launch", heads);
  const dim3 grid(tokens, heads);
  hipStream_t s = (hipStream_t)stream;
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  const bool based = (uintptr_t)pages % 16 == 0;
  const int key_vec = based && dim % vec == 0 && ((int64_t)vdim * page_size) % vec == 0;
  const bool paged_vec = based && WAVE % page_size == 0 && page_size % vec == 0;
#define SMX_LAUNCH(T, PV)                                                                                            \
  softmax_attention_kernel<T, PV><<<grid, 256, 0, s>>>((const T*)q, (T*)out, (const T*)pages, table, table_stride,   \
                                                       table_rows, slots, token_row, positions, heads, kv_heads, dim, \
                                                       vdim, page_size, num_pages, sink, scale, window, key_vec)
  if (dtype == HOLON_F32) { if (paged_vec) SMX_LAUNCH(float, true); else SMX_LAUNCH(float, false); }
  else { if (paged_vec) SMX_LAUNCH(bf16_t, true); else SMX_LAUNCH(bf16_t, false); }
#undef SMX_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}
