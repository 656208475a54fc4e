// A residual stream kept in float32: the kernels around it. Terms in the engine's dtype (or float32) are added into
// float32 rows and the layer norm that reads the sum runs in the same kernel; every sum over a row is taken in an order
// that the row's width alone decides, so a token's result does not depend on what else is in the batch.
#include "common.h"
#include "holon_hip.h"

namespace {

__device__ __forceinline__ float load_as(const void* p, int64_t i, int dt) {
  return dt == HOLON_F32 ? reinterpret_cast<const float*>(p)[i] : bf16_to_float(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void store_as(void* p, int64_t i, int dt, float v) {
  if (dt == HOLON_F32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<bf16_t*>(p)[i] = float_to_bf16(v);
}

// Sum over a block of 256 threads, every thread gets the result; waves are added in order.
__device__ __forceinline__ float block_sum_256(float v, float* part) {
  v = wave_sum(v);
  __syncthreads();                       // `part` may still be read from the call before
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = v;
  __syncthreads();
  return (part[0] + part[1]) + (part[2] + part[3]);
}

__global__ void widen_kernel(const void* __restrict__ x, float* __restrict__ y, int64_t n, int dt) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    y[i] = load_as(x, i, dt);
}

// One block a row: x += s1 d1 + s2 d2 (either may be absent); then, with a weight, y = (x - mean) / sqrt(var + eps) * w
// with the variance taken about the mean in a second pass over the row. REGS: the row (up to 256 * REGS values) stays in
// registers between the passes; 0: it is read back from memory (a thread reads what it wrote itself).
template <int REGS>
__global__ void __launch_bounds__(256) stream_norm_kernel(float* __restrict__ x32, const void* __restrict__ d1, float s1,
                                                          int dt1, const void* __restrict__ d2, float s2, int dt2,
                                                          const void* __restrict__ weight, void* __restrict__ y, int dim,
                                                          float eps, int dt_out) {
  __shared__ float part[4];
  const int64_t base = (int64_t)blockIdx.x * dim;
  float* x = x32 + base;
  float sum = 0.f;
  float held[REGS > 0 ? REGS : 1];
  auto updated = [&](int i) {
    float v = x[i];
    if (d1) v += s1 * load_as(d1, base + i, dt1);
    if (d2) v += s2 * load_as(d2, base + i, dt2);
    if (d1 || d2) x[i] = v;
    return v;
  };
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      held[e] = i < dim ? updated(i) : 0.f;
      sum += held[e];
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) sum += updated(i);
  }
  if (!weight) return;
  const float mean = block_sum_256(sum, part) / (float)dim;
  float sq = 0.f;
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const float d = threadIdx.x + e * 256 < dim ? held[e] - mean : 0.f;
      sq += d * d;
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) {
      const float d = x[i] - mean;
      sq += d * d;
    }
  }
  const float var = block_sum_256(sq, part) / (float)dim;
  const float r = 1.0f / sqrtf(var + eps);
  if constexpr (REGS > 0) {
#pragma unroll
    for (int e = 0; e < REGS; ++e) {
      const int i = threadIdx.x + e * 256;
      if (i < dim) store_as(y, base + i, dt_out, (held[e] - mean) * r * load_as(weight, i, dt_out));
    }
  } else {
    for (int i = threadIdx.x; i < dim; i += 256) store_as(y, base + i, dt_out, (x[i] - mean) * r * load_as(weight, i, dt_out));
  }
}

__global__ void pair_rows_kernel(const float* __restrict__ x32, const void* __restrict__ origin, void* __restrict__ y,
                                 int64_t rows, int w1, int w2, int dt_origin, int dt_out) {
  const int64_t n = rows * (w1 + w2);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / (w1 + w2);
    const int c = (int)(i - row * (w1 + w2));
    const float v = c < w1 ? x32[row * w1 + c] : load_as(origin, row * w2 + (c - w1), dt_origin);
    store_as(y, i, dt_out, v);
  }
}

__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] / cap);
}

inline int blocks_for(int64_t n) { return (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535); }
}  // namespace

extern "C" int holon_widen_rows(const void* x, float* y, int64_t n, int dtype, void* stream) {
  HOLON_CHECK(n >= 0 && (dtype == HOLON_F32 || dtype == HOLON_BF16), "widen_rows: n=%lld dtype=%d", (long long)n, dtype);
  if (n == 0) return 0;
  widen_kernel<<<blocks_for(n), 256, 0, (hipStream_t)stream>>>(x, y, n, dtype);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_stream_norm(float* x32, const void* d1, float s1, int dt1, const void* d2, float s2, int dt2,
                                 const void* weight, void* y, int64_t rows, int dim, float eps, int dt_out,
                                 void* stream) {
  HOLON_CHECK(rows >= 0 && dim > 0 && (weight == nullptr) == (y == nullptr), "stream_norm: rows=%lld dim=%d",
              (long long)rows, dim);
  HOLON_CHECK(rows <= 0x7fffffff, "stream_norm: %lld rows exceed one launch", (long long)rows);
  if (rows == 0 || (!d1 && !d2 && !weight)) return 0;
  if (!d1 && d2) { d1 = d2; s1 = s2; dt1 = dt2; d2 = nullptr; }
#define NORM_LAUNCH(REGS) \
  stream_norm_kernel<REGS><<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>(x32, d1, s1, dt1, d2, s2, dt2, weight, y, dim, \
                                                                            eps, dt_out)
  if (dim <= 1024) NORM_LAUNCH(4);          // (the sums' order is the same in every form: a thread's values in
  else if (dim <= 2048) NORM_LAUNCH(8);     // ascending order, then the block's)
  else if (dim <= 4096) NORM_LAUNCH(16);
  else NORM_LAUNCH(0);
#undef NORM_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_pair_rows(const float* x32, const void* origin, void* y, int64_t rows, int w1, int w2,
                               int dt_origin, int dt_out, void* stream) {
  HOLON_CHECK(rows >= 0 && w1 > 0 && w2 > 0, "pair_rows: rows=%lld widths %d, %d", (long long)rows, w1, w2);
  if (rows == 0) return 0;
  pair_rows_kernel<<<blocks_for(rows * (w1 + w2)), 256, 0, (hipStream_t)stream>>>(x32, origin, y, rows, w1, w2,
                                                                                  dt_origin, dt_out);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_softcap(float* logits, int64_t n, float cap, void* stream) {
  HOLON_CHECK(n >= 0 && cap > 0.f, "softcap: n=%lld cap=%g", (long long)n, (double)cap);
  if (n == 0) return 0;
  softcap_kernel<<<blocks_for(n), 256, 0, (hipStream_t)stream>>>(logits, n, cap);
  HOLON_LAUNCH_OK();
  return 0;
}
