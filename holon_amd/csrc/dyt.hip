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

template <typename TX, typename TT, typename TY>
__global__ void __launch_bounds__(256) dyt_stream_kernel(TX* __restrict__ x, const TT* __restrict__ term, DytNorm post,
                                                         float scale, const float* __restrict__ extra, DytNorm pre,
                                                         TY* __restrict__ y, int64_t cells, int dim) {
  const float a1 = term ? post.alpha[0] : 0.f;
  const float a2 = y ? pre.alpha[0] : 0.f;
  // a thread takes four neighbouring values of a row (the host sees to it that dim is a multiple of 4, or passes
  // cells as single values with dim as it is: then `quad` is 1)
  const int quad = (dim % 4 == 0) ? 4 : 1;
  const int64_t n = cells / quad;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t at = i * quad;
    const int c = (int)(at % dim);
#pragma unroll 4
    for (int e = 0; e < quad; ++e) {
      float v = Elem<TX>::load(x[at + e]);
      if (term) v += scale * (tanhf(a1 * Elem<TT>::load(term[at + e])) * post.w[c + e] + post.b[c + e]);
      if (extra) v += extra[at + e];
      if (term || extra) x[at + e] = Elem<TX>::store(v);
      if (y) y[at + e] = Elem<TY>::store(tanhf(a2 * v) * pre.w[c + e] + pre.b[c + e]);
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
  const int64_t threads = dim % 4 == 0 ? cells / 4 : cells;
  const int64_t want = (threads + 255) / 256;
  const unsigned blocks = (unsigned)(want < 1 ? 1 : want > 16384 ? 16384 : want);
  const DytNorm post{post_alpha, post_w, post_b}, pre{pre_alpha, pre_w, pre_b};
  hipStream_t s = (hipStream_t)stream;
#define DYT_LAUNCH(TX, TT, TY) \
  dyt_stream_kernel<TX, TT, TY><<<blocks, 256, 0, s>>>((TX*)x, (const TT*)term, post, scale, extra, pre, (TY*)y, cells, dim)
#define DYT_BY_Y(TX, TT) do { if (y_dtype == HOLON_F32) DYT_LAUNCH(TX, TT, float); else DYT_LAUNCH(TX, TT, bf16_t); } while (0)
  if (x_dtype == HOLON_F32) {
    if (term_dtype == HOLON_F32) DYT_BY_Y(float, float); else DYT_BY_Y(float, bf16_t);
  } else {
    DYT_BY_Y(bf16_t, bf16_t);              // nothing is added: the rows are only read
  }
#undef DYT_BY_Y
#undef DYT_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}
