// A matrix memory with exponential gates (the mLSTM cell of xLSTM), carried from token to token per
// sequence and head. With q (already times dim^-1/2), k of width D, v of width Dv, a log input gate i
// and a log forget gate f per token and head:
//
//   i = cap * tanh((a_i + b_i) / cap),  f = logsigmoid(cap * tanh((a_f + b_f) / cap))     (a: the gates' projections)
//   m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
//
// S [D, Dv], n [D] and m live in float32 in the state store (zero when a sequence starts, so m starts
// at 0) and everything above is float arithmetic. A second kernel divides each head's o by its root mean
// square, multiplies by a weight over all heads' features and by sigmoid(g), and rounds once.
//
// The recurrence kernel walks a sequence's rows of the step in order, whatever their number: a prompt, a
// further portion of one, or one token. Grid (sequence, head, run of 63 value columns). A workgroup holds
// its columns of S in registers, one column a lane, the rows of S dealt to its waves; lane 63 holds n as
// one more column whose "value" is 1, so the same multiply-adds update it and the same reduction gives
// n . q. Tokens are staged through LDS a tile at a time.
#include "common.h"

#define MLSTM_COLS 63            // value columns a workgroup owns; lane 63 is the normaliser's
#define MLSTM_TILE 16            // tokens staged at a time
#define MLSTM_MAX_WAVES 16
#define MLSTM_MAX_HELD 16        // rows of S a thread may hold: D <= waves * this

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T, int HELD>
__global__ __launch_bounds__(1024) void mlstm_steps_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_col, int k_col, int v_col,
    const float* __restrict__ gates, const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state_s, float* __restrict__ state_n, float* __restrict__ state_m,
    float* __restrict__ o_raw, int n_heads, int dim, int v_dim, float q_scale, int write_state) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, head = blockIdx.y, c0 = blockIdx.z * MLSTM_COLS;
  const int slot = seq_slot[seq];
  if (slot < 0) return;                                   // the sequence sits out: its rows of o_raw are not read
  const int waves = blockDim.x / WAVE, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int row0 = cu_rows[seq], n_tok = q_len[seq];
  const int col = c0 + lane;
  const bool is_n = lane == MLSTM_COLS, is_v = !is_n && col < v_dim;
  float* qs = lds;                                        // [TILE][dim]
  float* ks = qs + MLSTM_TILE * dim;                      // [TILE][dim]
  float* vs = ks + MLSTM_TILE * dim;                      // [TILE][64]: the workgroup's columns, 1 in the last
  float* gi = vs + MLSTM_TILE * WAVE;                     // [TILE]
  float* gf = gi + MLSTM_TILE;                            // [TILE]
  float* red = gf + MLSTM_TILE;                           // [2][waves][64]
  const int64_t sh = (int64_t)slot * n_heads + head;
  float* S = state_s + sh * dim * v_dim;
  float* N = state_n + sh * dim;
  float held[HELD];
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int d = wave + j * waves;
    held[j] = d < dim ? (is_n ? N[d] : (is_v ? S[(int64_t)d * v_dim + col] : 0.f)) : 0.f;
  }
  float m = state_m[sh];
  for (int t0 = 0; t0 < n_tok; t0 += MLSTM_TILE) {
    const int nt = min(MLSTM_TILE, n_tok - t0);
    __syncthreads();                                      // the tile before is no longer read
    for (int e = threadIdx.x; e < nt * dim; e += blockDim.x) {
      const int t = e / dim, d = e % dim;
      const T* p = proj + (int64_t)(row0 + t0 + t) * proj_stride + (int64_t)head * dim + d;
      qs[e] = load_as_float(p + q_col) * q_scale;
      ks[e] = load_as_float(p + k_col);
    }
    for (int e = threadIdx.x; e < nt * WAVE; e += blockDim.x) {
      const int t = e / WAVE, l = e % WAVE, c = c0 + l;
      float v = 0.f;
      if (l == MLSTM_COLS) v = 1.f;
      else if (c < v_dim) v = load_as_float(proj + (int64_t)(row0 + t0 + t) * proj_stride + v_col + (int64_t)head * v_dim + c);
      vs[e] = v;
    }
    if (threadIdx.x < nt) {
      const float* g = gates + (int64_t)(row0 + t0 + threadIdx.x) * 2 * n_heads;
      gi[threadIdx.x] = cap * tanhf((g[head] + bias_i[head]) / cap);
      gf[threadIdx.x] = log_sigmoid(cap * tanhf((g[n_heads + head] + bias_f[head]) / cap));
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float m_new = fmaxf(gf[t] + m, gi[t]);
      const float keep = expf(gf[t] + m - m_new), take = expf(gi[t] - m_new);
      m = m_new;
      const float tv = take * vs[t * WAVE + lane];
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < HELD; ++j) {
        const int d = wave + j * waves;
        if (d < dim) {
          held[j] = keep * held[j] + ks[t * dim + d] * tv;
          part += held[j] * qs[t * dim + d];
        }
      }
      float* r = red + ((t0 + t) & 1) * waves * WAVE;
      r[wave * WAVE + lane] = part;
      __syncthreads();                                    // one barrier a token: the two halves of `red` take turns
      if (wave == 0) {
        float tot = 0.f;
        for (int w = 0; w < waves; ++w) tot += r[w * WAVE + lane];
        const float nq = __shfl(tot, MLSTM_COLS, WAVE);
        const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
        if (is_v) o_raw[((int64_t)(row0 + t0 + t) * n_heads + head) * v_dim + col] = tot / den;
      }
    }
  }
  if (!write_state) return;
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int d = wave + j * waves;
    if (d < dim) {
      if (is_n) { if (blockIdx.z == 0) N[d] = held[j]; }
      else if (is_v) S[(int64_t)d * v_dim + col] = held[j];
    }
  }
  if (blockIdx.z == 0 && threadIdx.x == 0) state_m[sh] = m;
}

DRYFT_API int dryft_mlstm_lds_bytes(int dim, int waves) {
  return (2 * MLSTM_TILE * dim + MLSTM_TILE * WAVE + 2 * MLSTM_TILE + 2 * waves * WAVE) * (int)sizeof(float);
}

// gates: float32 [rows, 2 * heads], the input gates' projections then the forget gates'. o_raw: float32
// [rows, heads, v_dim]. The state tensors are indexed by slot.
DRYFT_API int dryft_mlstm_steps(const void* proj, int64_t proj_stride, int q_col, int k_col, int v_col,
                                const float* gates, const float* bias_i, const float* bias_f, float cap,
                                const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs, float* state_s,
                                float* state_n, float* state_m, float* o_raw, int n_heads, int dim, int v_dim,
                                float q_scale, int write_state, int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (dim <= 0 || v_dim <= 0 || dim > MLSTM_MAX_WAVES * MLSTM_MAX_HELD || !(cap > 0.f)) return -1;
  int waves = 4;                                          // as many waves as keep a thread's rows of S few
  while (waves < MLSTM_MAX_WAVES && waves * 4 < dim) waves *= 2;
  const int held = (dim + waves - 1) / waves;
  const int lds = dryft_mlstm_lds_bytes(dim, waves);
  if (lds > 64 * 1024) return -1;
  dim3 grid(n_seqs, n_heads, (v_dim + MLSTM_COLS - 1) / MLSTM_COLS), block(waves * WAVE);
#define ML(TT, HH)                                                                                                   \
  hipLaunchKernelGGL((mlstm_steps_kernel<TT, HH>), grid, block, lds, stream, (const TT*)proj, proj_stride, q_col,    \
                     k_col, v_col, gates, bias_i, bias_f, cap, seq_slot, cu_rows, q_len, state_s, state_n, state_m,  \
                     o_raw, n_heads, dim, v_dim, q_scale, write_state)
#define ML_T(HH) do { if (is_f32) ML(float, HH); else ML(bf16_t, HH); } while (0)
  if (held <= 4) ML_T(4);
  else if (held <= 8) ML_T(8);
  else ML_T(16);
#undef ML_T
#undef ML
  return DRYFT_LAUNCH_CHECK();
}

// out[row, head * v_dim + c] = T( o / sqrt(mean_c(o^2) + eps) * w[head * v_dim + c] * sigmoid(g) ): each head's
// output divided by its root mean square, weighted, gated. One wave a (row, head); rows of sequences that sit
// out get zeros.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ proj,
                                                        int64_t proj_stride, int g_col, const float* __restrict__ w,
                                                        const int* __restrict__ row_slot, T* __restrict__ out,
                                                        int n_heads, int v_dim, float eps) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t row = blockIdx.x;
  const int head = blockIdx.y * 4 + wave;
  if (head >= n_heads) return;
  T* dst = out + (row * n_heads + head) * v_dim;
  if (row_slot[row] < 0) {
    for (int c = lane; c < v_dim; c += WAVE) store_from_float(dst + c, 0.f);
    return;
  }
  const float* o = o_raw + (row * n_heads + head) * v_dim;
  float ss = 0.f;
  for (int c = lane; c < v_dim; c += WAVE) ss += o[c] * o[c];
  const float inv = rsqrtf(wave_sum(ss) / (float)v_dim + eps);
  const T* g = proj + row * proj_stride + g_col + (int64_t)head * v_dim;
  for (int c = lane; c < v_dim; c += WAVE) {
    const float gate = 1.f / (1.f + expf(-load_as_float(g + c)));
    store_from_float(dst + c, o[c] * inv * w[head * v_dim + c] * gate);
  }
}

DRYFT_API int dryft_mlstm_out(const float* o_raw, const void* proj, int64_t proj_stride, int g_col, const float* w,
                              const int* row_slot, void* out, int n_rows, int n_heads, int v_dim, float eps,
                              int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  dim3 grid(n_rows, (n_heads + 3) / 4), block(256);
  if (is_f32)
    hipLaunchKernelGGL(mlstm_out_kernel<float>, grid, block, 0, stream, o_raw, (const float*)proj, proj_stride, g_col,
                       w, row_slot, (float*)out, n_heads, v_dim, eps);
  else
    hipLaunchKernelGGL(mlstm_out_kernel<bf16_t>, grid, block, 0, stream, o_raw, (const bf16_t*)proj, proj_stride,
                       g_col, w, row_slot, (bf16_t*)out, n_heads, v_dim, eps);
  return DRYFT_LAUNCH_CHECK();
}
