// The matrix memory of xLSTM (mLSTM) along each row's tokens. Per (row, head): a matrix S [D, V], a vector n [D] and a
// running maximum m, float32, carried in the request's slot (a row that starts at position 0 starts from S = 0, n = 0
// and a maximum of 0, whatever the slot holds). With log gates i and f of the token:
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' = exp(f + m - m') n + exp(i - m') k
//   o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// The gates come as pre-activations a of a projection and a bias: i = cap tanh((a_i + b_i) / cap),
// f = logsigmoid(cap tanh((a_f + b_f) / cap)); q is scaled by D^-0.5. q, k, v and the gates are columns of one
// projection's rows.
//
// n is kept as one more column of S (the column of a value that is always 1), so the state is S [D, V + 1] and the
// kernel leaves the numerators S'^T q [V] and the denominator max(|n' . q|, exp(-m')) + 1e-6 of every token; the
// read-out kernel that follows divides. S's columns never meet, so a wave owns 8 of them, eight lanes a column with an
// eighth of the key rows each; what a token needs of a whole column is summed over a lane's rows in four interleaved
// chains and then over the eight lanes in a fixed order. A batch of tokens' operands travels from memory to LDS while
// the batch before is worked through; the gates' functions are taken then, off the recurrence's path.
// The blocks of a head (one for every 8 columns) all need m and do not wait for each other, so each keeps a copy of
// its own in the slot, m [H, ceil((V + 1) / 8)]: a block reads and writes nothing that another block touches.
//
// Long rows run in pieces side by side. The maxima depend on the gates alone, m' = max(m + f, i), a recurrence whose
// steps compose ((a, b) then (c, d) is (a + c, max(b + c, d))), so a wave finds a whole row's maxima by a prefix scan and
// leaves every token's two factors exp(f + m - m') and exp(i - m') and exp(-m') behind. With those the recurrence is
// linear in S and n with factors that do not depend on them: every piece but a row's last first runs from zero and
// leaves what it adds and the product of its factors; a small kernel walks a row's pieces in order, leaving each
// piece's true start; then every piece runs again from there and writes its outputs.
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

struct MlstmPieces {
  int tokens;                  // tokens a piece (0: rows are not cut, the gates are taken inside the scan)
  int mode;                    // 1: from zero, leave what the piece adds; 2: from the true start, write outputs
  const int32_t* base;         // [rows]: the number of row b's first piece among all pieces of the step
  const float* gates;          // [T, H, 3]: exp(f + m - m'), exp(i - m'), exp(-m') of every token
  float* sloc;                 // [pieces, H, D, V + 1]
  float* pk;                   // [pieces, H]
};

// One wave per (row, head): the row's maxima by a prefix scan over lanes that each hold a run of neighbouring tokens,
// then every token's three factors. The slot's copies of m take the row's last maximum.
template <typename T>
__global__ void __launch_bounds__(WAVE) mlstm_gates_kernel(const T* __restrict__ proj, int width, int gate_off,
                                                           const float* __restrict__ gate_bias, float cap,
                                                           float* __restrict__ m_all, float* __restrict__ gates,
                                                           const int32_t* __restrict__ slots,
                                                           const int32_t* __restrict__ starts,
                                                           const int32_t* __restrict__ query_start, int heads,
                                                           int copies) {
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int lo = query_start[b], hi = query_start[b + 1], n = hi - lo;
  if (n <= 0) return;
  const int64_t cell = ((int64_t)slots[b] * heads + h) * copies;
  const float m0 = starts[b] > 0 ? m_all[cell] : 0.f;
  const float bi = gate_bias[h], bf = gate_bias[heads + h];
  const int seg = (n + WAVE - 1) / WAVE;
  const int t0 = lo + lane * seg, t1 = min(hi, t0 + seg);
  auto gate = [&](int t, float& it, float& ft) {
    const T* row = proj + (int64_t)t * width + gate_off;
    it = cap * tanhf((Elem<T>::load(row[h]) + bi) / cap);
    ft = log_sigmoid(cap * tanhf((Elem<T>::load(row[heads + h]) + bf) / cap));
  };
  float A = 0.f, B = -INFINITY;                       // this lane's run as one step: m -> max(m + A, B)
  for (int t = t0; t < t1; ++t) {
    float it, ft;
    gate(t, it, ft);
    B = fmaxf(B + ft, it);
    A += ft;
  }
#pragma unroll
  for (int off = 1; off < WAVE; off <<= 1) {           // inclusive scan: the runs of lanes 0 .. lane as one step
    const float Ao = __shfl_up(A, off, WAVE), Bo = __shfl_up(B, off, WAVE);
    if (lane >= off) {
      B = fmaxf(Bo + A, B);
      A = Ao + A;
    }
  }
  const float Ae = __shfl_up(A, 1, WAVE), Be = __shfl_up(B, 1, WAVE);
  float m = lane == 0 ? m0 : fmaxf(m0 + Ae, Be);
  for (int t = t0; t < t1; ++t) {
    float it, ft;
    gate(t, it, ft);
    const float m_new = fmaxf(ft + m, it);
    float* g = gates + ((int64_t)t * heads + h) * 3;
    g[0] = expf(ft + m - m_new);
    g[1] = expf(it - m_new);
    g[2] = expf(-m_new);
    m = m_new;
  }
  if (t0 < hi && t1 == hi)
    for (int c = 0; c < copies; ++c) m_all[cell + c] = m;
}

// A row's pieces in order: S <- pk S + sloc; sloc[p] becomes the state piece p + 1 starts from.
__global__ void __launch_bounds__(256) mlstm_pieces_kernel(const float* __restrict__ S_all,
                                                           const int32_t* __restrict__ slots,
                                                           const int32_t* __restrict__ starts,
                                                           const int32_t* __restrict__ query_start, int heads, int cells,
                                                           MlstmPieces pc) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int n = query_start[b + 1] - query_start[b];
  const int pieces = (n + pc.tokens - 1) / pc.tokens;
  if (pieces < 2) return;
  const int64_t cell = (int64_t)slots[b] * heads + h;
  const bool carried = starts[b] > 0;
  const int64_t first = pc.base[b];
  for (int e = blockIdx.z * 256 + threadIdx.x; e < cells; e += gridDim.z * 256) {
    float x = carried ? S_all[cell * cells + e] : 0.f;
    for (int p = 0; p < pieces - 1; ++p) {
      const int64_t at = (first + p) * heads + h;
      float* add = pc.sloc + at * cells + e;
      x = pc.pk[at] * x + *add;
      *add = x;
    }
  }
}

template <int KD, typename T>
__global__ void __launch_bounds__(WAVE) mlstm_scan_kernel(const T* __restrict__ proj, int width, int q_off, int k_off,
                                                          int v_off, int gate_off, const float* __restrict__ gate_bias,
                                                          float cap, float* __restrict__ S_all, float* __restrict__ m_all,
                                                          float* __restrict__ out, float* __restrict__ den_out,
                                                          const int32_t* __restrict__ slots,
                                                          const int32_t* __restrict__ starts,
                                                          const int32_t* __restrict__ query_start, int heads, int dim,
                                                          int vdim, int col_blocks, MlstmPieces pc) {
  constexpr int KQ = KD / PARTS, TC = KD <= 64 ? 16 : KD <= 128 ? 8 : 4, N = TC * KD, PER = (N + WAVE - 1) / WAVE;
  __shared__ float qs[2][N], ks[2][N];
  __shared__ float vs[2][TC * COLS], gi[2][TC], gf[2][TC], ge[2][TC];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int piece = blockIdx.z / col_blocks, col_block = blockIdx.z % col_blocks;
  const int part = lane % PARTS, col = lane / PARTS, j = col_block * COLS + col;
  const int cols = vdim + 1;                           // S's columns: the values', then n's
  const bool active = j < cols, of_n = j == vdim;
  int lo = query_start[b], hi = query_start[b + 1];
  const bool cut = pc.tokens > 0;                      // (the gates then come as factors: gi = keep, gf = take, ge = exp(-m))
  bool from_slot = true, to_slot = true;
  int64_t piece_no = 0;
  if (cut) {                                           // (everything here is the same in all of the block's lanes)
    const int pieces = (hi - lo + pc.tokens - 1) / pc.tokens;
    if (piece >= pieces || (pc.mode == 1 && piece == pieces - 1)) return;
    lo += piece * pc.tokens;
    hi = min(hi, lo + pc.tokens);
    from_slot = piece == 0;
    to_slot = pc.mode == 2 && piece == pieces - 1;
    piece_no = pc.base[b] + piece;
  }
  const bool local = cut && pc.mode == 1;
  const int64_t cell = (int64_t)slots[b] * heads + h;
  const int64_t mine = cell * col_blocks + col_block;        // this block's own copy of m
  float* S_held = S_all + cell * dim * cols;
  const bool carried = starts[b] > 0;
  float S[KQ];
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    if (local) {
      S[i] = 0.f;
    } else if (from_slot) {
      S[i] = (carried && active && row < dim) ? S_held[(int64_t)row * cols + j] : 0.f;
    } else {
      const int64_t at = (piece_no - 1) * heads + h;
      S[i] = (active && row < dim) ? pc.sloc[at * dim * cols + (int64_t)row * cols + j] : 0.f;
    }
  }
  float m = (carried && !cut) ? m_all[mine] : 0.f;
  float pk = 1.f;
  const float q_scale = 1.0f / sqrtf((float)dim);
  const float bi = gate_bias[h], bf = gate_bias[heads + h];
  float nq[PER], nk[PER], ngi = 0.f, ngf = 0.f, nge = 0.f;
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
      if (cut) {
        const float* g = pc.gates + ((int64_t)(t0 + lane) * heads + h) * 3;
        ngi = g[0];
        ngf = g[1];
        nge = g[2];
      } else {
        const T* row = proj + (int64_t)(t0 + lane) * width;
        const float ai = Elem<T>::load(row[gate_off + h]) + bi, af = Elem<T>::load(row[gate_off + heads + h]) + bf;
        ngi = cap * tanhf(ai / cap);
        ngf = log_sigmoid(cap * tanhf(af / cap));
      }
    }
  };
  float nv2[2];
  auto ask_v = [&](int t0) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int idx = lane + e * WAVE, tt = idx / COLS, jj = col_block * COLS + idx % COLS;
      const bool ok = idx < TC * COLS && t0 + tt < hi && jj < vdim;
      nv2[e] = ok ? Elem<T>::load(proj[(int64_t)(t0 + tt) * width + v_off + h * vdim + jj]) : (jj == vdim ? 1.f : 0.f);
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
    if (lane < TC) { gi[buf][lane] = ngi; gf[buf][lane] = ngf; ge[buf][lane] = nge; }
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
      float keep, take, floor_;
      if (cut) {
        keep = gi[buf][tt];
        take = gf[buf][tt];
        floor_ = ge[buf][tt];
      } else {
        const float it = gi[buf][tt], ft = gf[buf][tt];
        const float m_new = fmaxf(ft + m, it);
        keep = expf(ft + m - m_new);
        take = expf(it - m_new);
        m = m_new;
        floor_ = expf(-m);
      }
      const float vt = vs[buf][tt * COLS + col] * take;
      const float* qt = &qs[buf][tt * KD + part * KQ];
      const float* kt = &ks[buf][tt * KD + part * KQ];
      if (local) {                       // what the piece adds, and the product of its factors; no output yet
#pragma unroll
        for (int i = 0; i < KQ; ++i) S[i] = keep * S[i] + kt[i] * vt;
        pk *= keep;
        continue;
      }
      float os[4] = {0.f, 0.f, 0.f, 0.f};              // four short chains of sums, not one long one
#pragma unroll
      for (int i = 0; i < KQ; ++i) {
        S[i] = keep * S[i] + kt[i] * vt;
        os[i % 4] += S[i] * qt[i];
      }
      const float o = part_sum((os[0] + os[1]) + (os[2] + os[3]));
      if (active && part == 0) {
        if (of_n) den_out[(int64_t)(t0 + tt) * heads + h] = fmaxf(fabsf(o), floor_) + 1e-6f;
        else out[((int64_t)(t0 + tt) * heads + h) * vdim + j] = o;
      }
    }
    if (t0 + TC < hi) put(buf ^ 1);
    __syncthreads();
  }
  if (lo >= hi) return;
  if (local) {
    const int64_t at = piece_no * heads + h;
#pragma unroll
    for (int i = 0; i < KQ; ++i) {
      const int row = part * KQ + i;
      if (row >= dim) continue;
      if (active) pc.sloc[at * dim * cols + (int64_t)row * cols + j] = S[i];
    }
    if (col_block == 0 && lane == 0) pc.pk[at] = pk;
    return;
  }
  if (!to_slot) return;
#pragma unroll
  for (int i = 0; i < KQ; ++i) {
    const int row = part * KQ + i;
    if (row >= dim) continue;
    if (active) S_held[(int64_t)row * cols + j] = S[i];
  }
  if (lane == 0 && !cut) m_all[mine] = m;              // (cut: the gates' kernel has left the row's last maximum)
}

template <typename T, int KD>
void launch_mlstm(dim3 grid, hipStream_t s, const void* proj, int width, int q_off, int k_off, int v_off, int gate_off,
                  const float* gate_bias, float cap, float* S, float* m, float* out, float* den, const int32_t* slots,
                  const int32_t* starts, const int32_t* qs, int heads, int dim, int vdim, int col_blocks, MlstmPieces pc) {
  mlstm_scan_kernel<KD, T><<<grid, WAVE, 0, s>>>((const T*)proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap, S, m,
                                                  out, den, slots, starts, qs, heads, dim, vdim, col_blocks, pc);
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
                                const float* gate_bias, float cap, float* S, float* m, float* out, float* den,
                                const int32_t* slots, const int32_t* starts, const int32_t* query_start, int rows,
                                int heads, int dim, int vdim, int state_slots, int dtype, int tokens, int piece_tokens,
                                int max_pieces, const int32_t* piece_base, float* gates, float* sloc, float* pk,
                                void* stream) {
  HOLON_CHECK(rows >= 0 && heads > 0 && heads <= 65535 && dim > 0 && dim <= 256 && vdim > 0 && state_slots > 0,
              "mlstm_scan: %d heads of %d/%d (keys of at most 256)", heads, dim, vdim);
  HOLON_CHECK(cap > 0.f && width > 0 && q_off >= 0 && k_off >= 0 && v_off >= 0 && gate_off >= 0 &&
                  q_off + heads * dim <= width && k_off + heads * dim <= width && v_off + heads * vdim <= width &&
                  gate_off + 2 * heads <= width,
              "mlstm_scan: columns do not lie within rows of %d", width);
  HOLON_CHECK(piece_tokens == 0 || (piece_tokens > 0 && max_pieces > 0 && piece_base && gates && sloc && pk),
              "mlstm_scan: rows in pieces of %d tokens need the pieces' table and workspaces", piece_tokens);
  if (rows == 0) return 0;
  const int col_blocks = (vdim + 1 + COLS - 1) / COLS;     // the values' columns and n's
  hipStream_t s = (hipStream_t)stream;
  MlstmPieces pc{piece_tokens, 0, piece_base, gates, sloc, pk};
#define MLSTM_SCAN(GRID)                                                                                                \
  do {                                                                                                                  \
    if (dtype == HOLON_F32)                                                                                             \
      MLSTM_BY_KEY(dim, (launch_mlstm<float, KD>(GRID, s, proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap, S, \
                                                 m, out, den, slots, starts, query_start, heads, dim, vdim, col_blocks, \
                                                 pc)));                                                                 \
    else                                                                                                                \
      MLSTM_BY_KEY(dim, (launch_mlstm<bf16_t, KD>(GRID, s, proj, width, q_off, k_off, v_off, gate_off, gate_bias, cap,  \
                                                  S, m, out, den, slots, starts, query_start, heads, dim, vdim,         \
                                                  col_blocks, pc)));                                                    \
    HOLON_LAUNCH_OK();                                                                                                  \
  } while (0)
  if (piece_tokens == 0) {
    HOLON_CHECK(col_blocks <= 65535, "mlstm_scan: values of %d exceed one launch", vdim);
    const dim3 grid(rows, heads, col_blocks);
    MLSTM_SCAN(grid);
    return 0;
  }
  HOLON_CHECK((int64_t)col_blocks * max_pieces <= 65535, "mlstm_scan: %d pieces a row exceed one launch", max_pieces);
  (void)tokens;
  if (dtype == HOLON_F32)
    mlstm_gates_kernel<float><<<dim3(rows, heads), WAVE, 0, s>>>((const float*)proj, width, gate_off, gate_bias, cap, m,
                                                                 gates, slots, starts, query_start, heads, col_blocks);
  else
    mlstm_gates_kernel<bf16_t><<<dim3(rows, heads), WAVE, 0, s>>>((const bf16_t*)proj, width, gate_off, gate_bias, cap, m,
                                                                  gates, slots, starts, query_start, heads, col_blocks);
  HOLON_LAUNCH_OK();
  const dim3 grid(rows, heads, col_blocks * max_pieces);
  pc.mode = 1;
  MLSTM_SCAN(grid);
  const int cells = dim * (vdim + 1);
  const int walkers = (cells + 1023) / 1024;                // blocks a (row, head): four of its values a thread
  mlstm_pieces_kernel<<<dim3(rows, heads, walkers), 256, 0, s>>>(S, slots, starts, query_start, heads, cells, pc);
  HOLON_LAUNCH_OK();
  pc.mode = 2;
  MLSTM_SCAN(grid);
#undef MLSTM_SCAN
  return 0;
}
