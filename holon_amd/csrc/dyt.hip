// The Dynamic Tanh norm, y = tanh(alpha x) w + b, with the residual adds around it. Nothing is summed over a row, so one
// elementwise kernel takes the stream's rows through everything that lies between two sublayers:
//   x += scale * (tanh(a1 term) w1 + b1)      the sublayer's result through the norm behind it (if a term is given)
//   x += extra                                 rows added once more (if given)
//   y  = tanh(a2 x) w2 + b2                    the norm in front of the next sublayer (if given)
// x is float32 whenever anything is added; all arithmetic is float32 and y is rounded once.
#include "common.h"
#include "holon_hip.h"

namespace {

struct DytNorm {
  const float* alpha;      // one value, on the device
  const float* w;
  const float* b;
};

// tanh for results that are rounded to bfloat16 or added into sums of order one: 1 - 2 / (1 + e^2x) with the hardware's
// exponential and reciprocal, within 3e-7 of the true value everywhere. float32 results take the library's tanhf.
template <bool FAST> __device__ __forceinline__ float tanh_of(float x) {
  if (!FAST) return tanhf(x);
  const float e = __expf(2.0f * fminf(fmaxf(x, -15.f), 15.f));
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
}

template <typename T> struct Quad;                      // four neighbouring values as one load or store
template <> struct Quad<float> { typedef float4 type; };
template <> struct Quad<bf16_t> { typedef ushort4 type; };
template <typename T> __device__ __forceinline__ void load4(const T* p, float (&v)[4]);
template <> __device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
  const float4 r = *reinterpret_cast<const float4*>(p);
  v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float (&v)[4]) {
  const ushort4 r = *reinterpret_cast<const ushort4*>(p);
  v[0] = bf16_to_float(r.x); v[1] = bf16_to_float(r.y); v[2] = bf16_to_float(r.z); v[3] = bf16_to_float(r.w);
}
template <typename T> __device__ __forceinline__ void store4(T* p, const float (&v)[4]);
template <> __device__ __forceinline__ void store4<float>(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float (&v)[4]) {
  ushort4 r;
  r.x = float_to_bf16(v[0]); r.y = float_to_bf16(v[1]); r.z = float_to_bf16(v[2]); r.w = float_to_bf16(v[3]);
  *reinterpret_cast<ushort4*>(p) = r;
}

// QUAD: rows are whole groups of four values on 16-byte borders, and a thread takes a group as one load; else a
// thread takes single values. FAST: see tanh_of.
template <typename TX, typename TT, typename TY, bool QUAD, bool FAST>
__global__ void __launch_bounds__(256) dyt_stream_kernel(TX* __restrict__ x, const TT* __restrict__ term, DytNorm post,
                                                         float scale, const float* __restrict__ extra, DytNorm pre,
                                                         TY* __restrict__ y, int64_t cells, int dim) {
  const float a1 = term ? post.alpha[0] : 0.f;
  const float a2 = y ? pre.alpha[0] : 0.f;
  constexpr int N = QUAD ? 4 : 1;
  const int64_t n = cells / N;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t at = i * N;
    const int c = (int)(at % dim);
    float v[4], tv[4], ev[4], w1[4], b1[4], w2[4], b2[4], out[4];
    if (QUAD) {
      load4<TX>(x + at, v);
      if (term) { load4<TT>(term + at, tv); load4<float>(post.w + c, w1); load4<float>(post.b + c, b1); }
      if (extra) load4<float>(extra + at, ev);
      if (y) { load4<float>(pre.w + c, w2); load4<float>(pre.b + c, b2); }
    } else {
      v[0] = Elem<TX>::load(x[at]);
      if (term) { tv[0] = Elem<TT>::load(term[at]); w1[0] = post.w[c]; b1[0] = post.b[c]; }
      if (extra) ev[0] = extra[at];
      if (y) { w2[0] = pre.w[c]; b2[0] = pre.b[c]; }
    }
#pragma unroll
    for (int e = 0; e < N; ++e) {
      if (term) v[e] += scale * (tanh_of<FAST>(a1 * tv[e]) * w1[e] + b1[e]);
      if (extra) v[e] += ev[e];
      if (y) out[e] = tanh_of<FAST>(a2 * v[e]) * w2[e] + b2[e];
    }
    if (QUAD) {
      if (term || extra) store4<TX>(x + at, v);
      if (y) store4<TY>(y + at, out);
    } else {
      if (term || extra) x[at] = Elem<TX>::store(v[0]);
      if (y) y[at] = Elem<TY>::store(out[0]);
    }
  }
}
}  // namespace

extern "C" int holon_dyt_stream(void* x, int x_dtype, const void* term, int term_dtype, const float* post_alpha,
                                const float* post_w, const float* post_b, float scale, const float* extra,
                                const float* pre_alpha, const float* pre_w, const float* pre_b, void* y, int y_dtype,
                                int64_t rows, int dim, void* stream) {
  HOLON_CHECK(rows >= 0 && dim > 0, "dyt_stream: rows=%lld dim=%d", (long long)rows, dim);
  HOLON_CHECK(!(term || extra) || x_dtype == HOLON_F32, "dyt_stream: terms are added into float32 rows");
  HOLON_CHECK(!term || (post_alpha && post_w && post_b), "dyt_stream: a term needs its norm");
  HOLON_CHECK(!y || (pre_alpha && pre_w && pre_b), "dyt_stream: an output needs its norm");
  if (rows == 0 || (!term && !extra && !y)) return 0;
  const int64_t cells = rows * dim;
  const bool quad = dim % 4 == 0 && (((uintptr_t)x | (uintptr_t)term | (uintptr_t)extra | (uintptr_t)y |
                                      (uintptr_t)post_w | (uintptr_t)post_b | (uintptr_t)pre_w | (uintptr_t)pre_b) % 16 == 0);
  // the quick tanh where nothing float32 is handed on: bfloat16 terms in, bfloat16 rows out
  const bool fast = (!y || y_dtype == HOLON_BF16) && (!term || term_dtype == HOLON_BF16);
  const int64_t threads = quad ? cells / 4 : cells;
  const int64_t want = (threads + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : want > 16384 ? 16384 : want);
  const DytNorm post{post_alpha, post_w, post_b}, pre{pre_alpha, pre_w, pre_b};
  hipStream_t s = (hipStream_t)stream;
#define DYT_FORM(TX, TT, TY, Q, F) \
  dyt_stream_kernel<TX, TT, TY, Q, F><<<blocks, 256, 0, s>>>((TX*)x, (const TT*)term, post, scale, extra, pre, (TY*)y, cells, dim)
#define DYT_LAUNCH(TX, TT, TY)                                                \
  do {                                                                        \
    if (quad && fast) DYT_FORM(TX, TT, TY, true, true);                       \
    else if (quad) DYT_FORM(TX, TT, TY, true, false);                         \
    else if (fast) DYT_FORM(TX, TT, TY, false, true);                         \
    else DYT_FORM(TX, TT, TY, false, false);                                  \
  } while (0)
#define DYT_BY_Y(TX, TT) do { if (y_dtype == HOLON_F32) DYT_LAUNCH(TX, TT, float); else DYT_LAUNCH(TX, TT, bf16_t); } while (0)
  if (x_dtype == HOLON_F32) {
    if (term_dtype == HOLON_F32) DYT_BY_Y(float, float); else DYT_BY_Y(float, bf16_t);
  } else {
    DYT_BY_Y(bf16_t, bf16_t);              // nothing is added: the rows are only read
  }
#undef DYT_BY_Y
#undef DYT_LAUNCH
#undef DYT_FORM
  HOLON_LAUNCH_OK();
  return 0;
}
