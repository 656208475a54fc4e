// Softmax attention over a paged cache whose keys and values may differ in width, with an optional sliding window and an
// optional sink (one scalar per head whose exponential joins the normaliser; nothing is read from the cache for it). The general kernel: any
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

// -- the latent attention's small steps ---------------------------------------------------------------------------------
namespace {

// One block a token. `both` [T, q_rank + kv_rank] holds the two latents' projections side by side. Each is divided by
// its root mean square (eps inside the root) and multiplied by its weight, float32 inside, one rounding: the first goes
// to `cq` [T, q_rank]; the second is the token's entry in the cache, stored twice in the page it belongs to, as a key
// (a row of [P, kv_rank]) and as a value (a column of [kv_rank, P]).
template <typename T>
__global__ void __launch_bounds__(256) latent_prepare_kernel(const T* __restrict__ both, int q_rank, int kv_rank,
                                                             const T* __restrict__ q_weight, const T* __restrict__ c_weight,
                                                             float eps, T* __restrict__ cq, T* __restrict__ pages,
                                                             const int32_t* __restrict__ write_page,
                                                             const int32_t* __restrict__ write_off, int page_size,
                                                             int num_pages) {
  __shared__ float part[2][4];
  const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* row = both + (int64_t)t * (q_rank + kv_rank);
  float sq = 0.f, sc = 0.f;
  for (int d = threadIdx.x; d < q_rank; d += 256) { const float v = Elem<T>::load(row[d]); sq += v * v; }
  for (int d = threadIdx.x; d < kv_rank; d += 256) { const float v = Elem<T>::load(row[q_rank + d]); sc += v * v; }
  sq = wave_sum(sq);
  sc = wave_sum(sc);
  if (lane == 0) { part[0][wave] = sq; part[1][wave] = sc; }
  __syncthreads();
  const float rq = 1.0f / sqrtf(((part[0][0] + part[0][1]) + (part[0][2] + part[0][3])) / (float)q_rank + eps);
  const float rc = 1.0f / sqrtf(((part[1][0] + part[1][1]) + (part[1][2] + part[1][3])) / (float)kv_rank + eps);
  for (int d = threadIdx.x; d < q_rank; d += 256)
    cq[(int64_t)t * q_rank + d] = Elem<T>::store(Elem<T>::load(row[d]) * rq * Elem<T>::load(q_weight[d]));
  const int page = write_page[t], off = write_off[t];
  if (page < 0 || page >= num_pages || off < 0 || off >= page_size) return;
  T* keys = pages + (int64_t)page * 2 * page_size * kv_rank;
  T* vals = keys + (int64_t)page_size * kv_rank;
  for (int d = threadIdx.x; d < kv_rank; d += 256) {
    const T c = Elem<T>::store(Elem<T>::load(row[q_rank + d]) * rc * Elem<T>::load(c_weight[d]));
    keys[(int64_t)off * kv_rank + d] = c;
    vals[(int64_t)d * page_size + off] = c;
  }
}

// y[t, h, b] = sum_a x[t, h, a] w[h, b, a] for steps of few rows: a block takes a head and 16 of its output columns,
// the rows' values of that head wait in LDS, and sixteen lanes share a column (each a sixteenth of A, in the order of
// the lane), added up in a fixed order. float32 sums, one rounding.
template <typename T>
__global__ void __launch_bounds__(256) head_linear_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          T* __restrict__ y, int rows, int heads, int A, int B) {
  extern __shared__ float xs[];                          // [rows, A]
  const int h = blockIdx.x, b = blockIdx.y * 16 + threadIdx.x / 16, part = threadIdx.x % 16;
  for (int i = threadIdx.x; i < rows * A; i += 256) {
    const int t = i / A, a = i - t * A;
    xs[i] = Elem<T>::load(x[((int64_t)t * heads + h) * A + a]);
  }
  __syncthreads();
  const T* wr = w + ((int64_t)h * B + (b < B ? b : 0)) * A;
  constexpr int VEC = Elem<T>::kVec;
  const bool wide = A % (16 * VEC) == 0 && (uintptr_t)w % 16 == 0;      // a lane's share as 16-byte loads
  for (int t0 = 0; t0 < rows; t0 += 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (wide) {
      for (int a = part * VEC; a < A; a += 16 * VEC) {
        const uint4 raw = *reinterpret_cast<const uint4*>(wr + a);
        const T* e = reinterpret_cast<const T*>(&raw);
        float wv[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) wv[i] = Elem<T>::load(e[i]);
#pragma unroll
        for (int r = 0; r < 8; ++r)
          if (t0 + r < rows) {
            const float* xr = xs + (t0 + r) * A + a;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[r] += xr[i] * wv[i];
          }
      }
    } else {
      for (int a = part; a < A; a += 16) {
        const float wv = Elem<T>::load(wr[a]);
#pragma unroll
        for (int r = 0; r < 8; ++r)
          if (t0 + r < rows) acc[r] += xs[(t0 + r) * A + a] * wv;
      }
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      float v = acc[r];
      v += __shfl_xor(v, 1, WAVE);
      v += __shfl_xor(v, 2, WAVE);
      v += __shfl_xor(v, 4, WAVE);
      v += __shfl_xor(v, 8, WAVE);
      if (part == 0 && b < B && t0 + r < rows) y[((int64_t)(t0 + r) * heads + h) * B + b] = Elem<T>::store(v);
    }
  }
}
}  // namespace

extern "C" int holon_latent_prepare(const void* both, int tokens, int q_rank, int kv_rank, const void* q_weight,
                                    const void* c_weight, float eps, void* cq, void* pages, const int32_t* write_page,
                                    const int32_t* write_off, int page_size, int num_pages, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && q_rank > 0 && kv_rank > 0 && page_size > 0 && num_pages > 0,
              "latent_prepare: latents of %d and %d, pages of %d", q_rank, kv_rank, page_size);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    latent_prepare_kernel<float><<<tokens, 256, 0, s>>>((const float*)both, q_rank, kv_rank, (const float*)q_weight,
                                                       (const float*)c_weight, eps, (float*)cq, (float*)pages,
                                                       write_page, write_off, page_size, num_pages);
  else
    latent_prepare_kernel<bf16_t><<<tokens, 256, 0, s>>>((const bf16_t*)both, q_rank, kv_rank, (const bf16_t*)q_weight,
                                                        (const bf16_t*)c_weight, eps, (bf16_t*)cq, (bf16_t*)pages,
                                                        write_page, write_off, page_size, num_pages);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_head_linear_rows(const void* x, const void* w, void* y, int rows, int heads, int A, int B,
                                      int dtype, void* stream) {
  HOLON_CHECK(rows >= 1 && rows <= 16 && heads > 0 && heads <= 65535 && A > 0 && B > 0 && (int64_t)rows * A * 4 <= 48 * 1024,
              "head_linear (few rows): %d rows, %d heads of %d -> %d", rows, heads, A, B);
  const dim3 grid(heads, (B + 15) / 16);
  const size_t lds = (size_t)rows * A * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    head_linear_kernel<float><<<grid, 256, lds, s>>>((const float*)x, (const float*)w, (float*)y, rows, heads, A, B);
  else
    head_linear_kernel<bf16_t><<<grid, 256, lds, s>>>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, rows, heads, A, B);
  HOLON_LAUNCH_OK();
  return 0;
}
