// The matrix memory of xLSTM (mLSTM) along each row's tokens. Per (row, head): a matrix S [D, V], a vector n [D] and a
// running maximum m, float32, carried in the request's slot (a row that starts at position 0 starts from S = 0, n = 0,
// m = 0 whatever the slot holds). With log gates i and f of the token:
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' = exp(f + m - m') n + exp(i - m') k
//   o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// The gates come as pre-activations a of a projection and a bias: i = cap tanh((a_i + b_i) / cap),
// f = logsigmoid(cap tanh((a_f + b_f) / cap)); q is scaled by D^-0.5. q, k, v and the gates are columns of one
// projection's rows.
//
// S's columns never meet, so a wave owns 8 of them, eight lanes a column with an eighth of the key rows each (n's rows
// likewise, held again by every column); what a token needs of a whole column is summed over a lane's rows in ascending
// order and then over the eight lanes in a fixed order. A batch of tokens' operands travels from memory to LDS while
// the batch before is worked through; the gates' functions are taken then, off the recurrence's path.
// The blocks of a head (one for every 8 columns) all need n and m and do not wait for each other, so each keeps a copy
// of its own in the slot, n [H, V/8, D] and m [H, V/8]: a block reads and writes nothing that another block touches.
#include "common.h"
#include "holon_hip.h"

namespace {

template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float part_sum(float v) {      // over the eight adjacent lanes of a column, a fixed order
  v += dpp_move<0xB1>(v);        // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);        // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);       // row_half_mirror
  return v;
}

constexpr int PARTS = 8;                 // lanes a value column is spread over
constexpr int COLS = WAVE / PARTS;       // value columns a wave owns

__device__ __forceinline__ float log_sigmoid(float x) {   // -softplus(-x), without overflow on either side
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

template <int KD, typename T>
__global__ void __launch_bounds__(WAVE) mlstm_scan_kernel(const T* __restrict__ proj, int width, int q_off, int k_off,
                                                          int v_off, int gate_off, const float* __restrict__ gate_bias,
                                                          float cap, float* __restrict__ S_all, float* __restrict__ n_all,
                                                          float* __restrict__ m_all, float* __restrict__ out,
                                                          const int32_t* __restrict__ slots,
                                                          const int32_t* __restrict__ starts,
                                                          const int32_t* __restrict__ query_start, int heads, int dim,
                                                          int vdim) {
  constexpr int KQ = KD / PARTS, TC = KD <= 64 ? 16 : KD <= 128 ? 8 : 4, N = TC * KD, PER = (N + WAVE - 1) / WAVE;
  __shared__ float qs[2][N], ks[2][N];
  __shared__ float vs[2][TC * COLS], gi[2][TC], gf[2][TC];
  const int b = blockIdx.x, h = blockIdx.y, col_block = blockIdx.z, lane = threadIdx.x;
  const int part = lane % PARTS, col = lane / PARTS, j = col_block * COLS + col;
  const bool active = j < vdim;
  const int lo = query_start[b], hi = query_start[b + 1];
  const int64_t cell = (int64_t)slots[b] * heads + h;
  const int64_t mine = cell * gridDim.z + col_block;         // this block's own copy of n and m
  float* S_held = S_all + cell * dim * vdim;
  float* n_held = n_all + mine * dim;
  const bool carried = starts[b] > 0;
  float S[KQ], nn[KQ];
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    S[i] = (carried && active && row < dim) ? S_held[(int64_t)row * vdim + j] : 0.f;
    nn[i] = (carried && row < dim) ? n_held[row] : 0.f;
  }
  float m = carried ? m_all[mine] : 0.f;
  const float q_scale = 1.0f / sqrtf((float)dim);
  const float bi = gate_bias[h], bf = gate_bias[heads + h];
  float nq[PER], nk[PER], ngi = 0.f, ngf = 0.f;
  auto ask = [&](int t0) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE, tt = idx / KD, i = idx - tt * KD;
      const bool ok = idx < N && t0 + tt < hi && i < dim;
      const T* row = proj + (int64_t)(t0 + tt) * width;
      nq[e] = ok ? Elem<T>::load(row[q_off + h * dim + i]) * q_scale : 0.f;
      nk[e] = ok ? Elem<T>::load(row[k_off + h * dim + i]) : 0.f;
    }
    static_assert(TC * COLS <= 2 * WAVE, "a lane stages at most two values of v");
    if (lane < TC && t0 + lane < hi) {
      const T* row = proj + (int64_t)(t0 + lane) * width;
      const float ai = Elem<T>::load(row[gate_off + h]) + bi, af = Elem<T>::load(row[gate_off + heads + h]) + bf;
      ngi = cap * tanhf(ai / cap);
      ngf = log_sigmoid(cap * tanhf(af / cap));
    }
  };
  float nv2[2];
  auto ask_v = [&](int t0) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int idx = lane + e * WAVE, tt = idx / COLS, jj = col_block * COLS + idx % COLS;
      const bool ok = idx < TC * COLS && t0 + tt < hi && jj < vdim;
      nv2[e] = ok ? Elem<T>::load(proj[(int64_t)(t0 + tt) * width + v_off + h * vdim + jj]) : 0.f;
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < N) { qs[buf][idx] = nq[e]; ks[buf][idx] = nk[e]; }
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int idx = lane + e * WAVE;
      if (idx < TC * COLS) vs[buf][idx] = nv2[e];
    }
    if (lane < TC) { gi[buf][lane] = ngi; gf[buf][lane] = ngf; }
  };
  if (lo < hi) {
    ask(lo);
    ask_v(lo);
    put(0);
  }
  __syncthreads();
  for (int t0 = lo, buf = 0; t0 < hi; t0 += TC, buf ^= 1) {
    if (t0 + TC < hi) {
      ask(t0 + TC);
      ask_v(t0 + TC);
    }
    const int nt = min(TC, hi - t0);
    for (int tt = 0; tt < nt; ++tt) {
      const float it = gi[buf][tt], ft = gf[buf][tt];
      const float m_new = fmaxf(ft + m, it);
      const float keep = expf(ft + m - m_new), take = expf(it - m_new);
      m = m_new;
      const float vt = vs[buf][tt * COLS + col] * take;
      const float* qt = &qs[buf][tt * KD + part * KQ];
      const float* kt = &ks[buf][tt * KD + part * KQ];
      float o = 0.f, d = 0.f;
#pragma unroll
      for (int i = 0; i < KQ; ++i) {
        S[i] = keep * S[i] + kt[i] * vt;
        nn[i] = keep * nn[i] + take * kt[i];
        o += S[i] * qt[i];
        d += nn[i] * qt[i];
      }
      o = part_sum(o);
      d = part_sum(d);
      const float den = fmaxf(fabsf(d), expf(-m)) + 1e-6f;
      if (active && part == 0) out[((int64_t)(t0 + tt) * heads + h) * vdim + j] = o / den;
    }
    if (t0 + TC < hi) put(buf ^ 1);
    __syncthreads();
  }
  if (lo >= hi) return;
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    if (row >= dim) continue;
    if (active) S_held[(int64_t)row * vdim + j] = S[i];
    if (col == 0) n_held[row] = nn[i];
  }
  if (lane == 0) m_all[mine] = m;
}

template <typename T, int KD>
void launch_mlstm(dim3 grid, hipStream_t s, const void* proj, int width, int q_off, int k_off, int v_off, int gate_off,
                  const float* gate_bias, float cap, float* S, float* n, float* m, float* out, const int32_t* slots,
                  const int32_t* starts, const int32_t* qs, int heads, int dim, int vdim) {
  mlstm_scan_kernel<KD, T><<<grid, WAVE, 0, s>>>((const T*)proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap, S, n,
                                                  m, out, slots, starts, qs, heads, dim, vdim);
}
}  // namespace

#define MLSTM_BY_KEY(dim, CALL)                               \
  do {                                                        \
    if ((dim) <= 16) { constexpr int KD = 16; CALL; }         \
    else if ((dim) <= 32) { constexpr int KD = 32; CALL; }    \
    else if ((dim) <= 64) { constexpr int KD = 64; CALL; }    \
    else if ((dim) <= 128) { constexpr int KD = 128; CALL; }  \
    else { constexpr int KD = 256; CALL; }                    \
  } while (0)

extern "C" int holon_mlstm_scan(const void* proj, int width, int q_off, int k_off, int v_off, int gate_off,
                                const float* gate_bias, float cap, float* S, float* n, float* m, float* out,
                                const int32_t* slots, const int32_t* starts, const int32_t* query_start, int rows,
                                int heads, int dim, int vdim, int state_slots, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && heads > 0 && heads <= 65535 && dim > 0 && dim <= 256 && vdim > 0 && state_slots > 0,
              "mlstm_scan: %d heads of %d/%d (keys of at most 256)", heads, dim, vdim);
  HOLON_CHECK(cap > 0.f && width > 0 && q_off >= 0 && k_off >= 0 && v_off >= 0 && gate_off >= 0 &&
                  q_off + heads * dim <= width && k_off + heads * dim <= width && v_off + heads * vdim <= width &&
                  gate_off + 2 * heads <= width,
              "mlstm_scan: columns do not lie within rows of %d", width);
  if (rows == 0) return 0;
  const int col_blocks = (vdim + COLS - 1) / COLS;
  HOLON_CHECK(col_blocks <= 65535, "mlstm_scan: values of %d exceed one launch", vdim);
  const dim3 grid(rows, heads, col_blocks);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    MLSTM_BY_KEY(dim, (launch_mlstm<float, KD>(grid, s, proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap, S, n,
                                               m, out, slots, starts, query_start, heads, dim, vdim)));
  else
    MLSTM_BY_KEY(dim, (launch_mlstm<bf16_t, KD>(grid, s, proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap, S,
                                                n, m, out, slots, starts, query_start, heads, dim, vdim)));
  HOLON_LAUNCH_OK();
  return 0;
}
