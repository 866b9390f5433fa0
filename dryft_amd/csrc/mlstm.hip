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
// further portion of one, or one token. Grid (sequence, head, run of 64 value columns). A workgroup holds
// its columns of S in registers, one column a lane, the rows of S dealt to its waves, and beside them n (every
// lane of a wave the same entries), whose product with q goes through the same reduction as one more column.
// Tokens are staged through LDS a tile at a time. n and m are kept once per run of 64 value columns
// ([.., heads, runs, D] and [.., heads, runs]): every workgroup reads and writes its own copy, so none ever
// reads what another has already updated.
#include "common.h"

#define MLSTM_COLS 64            // value columns a workgroup owns
#define MLSTM_RED (MLSTM_COLS + 1)  // a wave's partial sums: its columns, then n . q
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
  const bool is_v = col < v_dim;
  const int runs = gridDim.z;
  float* qs = lds;                                        // [TILE][dim]
  float* ks = qs + MLSTM_TILE * dim;                      // [TILE][dim]
  float* vs = ks + MLSTM_TILE * dim;                      // [TILE][64]: the workgroup's columns
  float* gi = vs + MLSTM_TILE * WAVE;                     // [TILE]
  float* gf = gi + MLSTM_TILE;                            // [TILE]
  float* red = gf + MLSTM_TILE;                           // [2][waves][65]
  const int64_t sh = (int64_t)slot * n_heads + head;
  float* S = state_s + sh * dim * v_dim;
  float* N = state_n + (sh * runs + blockIdx.z) * dim;
  float held[HELD], held_n[HELD];
#pragma unroll
  for (int j = 0; j < HELD; ++j) {
    const int d = wave + j * waves;
    held[j] = (d < dim && is_v) ? S[(int64_t)d * v_dim + col] : 0.f;
    held_n[j] = d < dim ? N[d] : 0.f;
  }
  float m = state_m[sh * runs + blockIdx.z];
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
      if (c < v_dim) v = load_as_float(proj + (int64_t)(row0 + t0 + t) * proj_stride + v_col + (int64_t)head * v_dim + c);
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
      float part = 0.f, part_n = 0.f;
#pragma unroll
      for (int j = 0; j < HELD; ++j) {
        const int d = wave + j * waves;
        if (d < dim) {
          held[j] = keep * held[j] + ks[t * dim + d] * tv;
          held_n[j] = keep * held_n[j] + ks[t * dim + d] * take;
          part += held[j] * qs[t * dim + d];
          part_n += held_n[j] * qs[t * dim + d];
        }
      }
      float* r = red + ((t0 + t) & 1) * waves * MLSTM_RED;
      r[wave * MLSTM_RED + lane] = part;
      if (lane == 0) r[wave * MLSTM_RED + MLSTM_COLS] = part_n;
      __syncthreads();                                    // one barrier a token: the two halves of `red` take turns
      if (wave == 0) {
        float tot = 0.f, nq = 0.f;
        for (int w = 0; w < waves; ++w) {
          tot += r[w * MLSTM_RED + lane];
          nq += r[w * MLSTM_RED + MLSTM_COLS];
        }
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
      if (is_v) S[(int64_t)d * v_dim + col] = held[j];
      if (lane == 0) N[d] = held_n[j];
    }
  }
  if (threadIdx.x == 0) state_m[sh * runs + blockIdx.z] = m;
}

DRYFT_API int dryft_mlstm_lds_bytes(int dim, int waves) {
  return (2 * MLSTM_TILE * dim + MLSTM_TILE * WAVE + 2 * MLSTM_TILE + 2 * waves * MLSTM_RED) * (int)sizeof(float);
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
                                                        int n_heads, int v_dim, float eps, int vec) {
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
  const T* g = proj + row * proj_stride + g_col + (int64_t)head * v_dim;
  if (vec) {                                               // 8 values a lane, 16 bytes a load (widths of 8 up to 512)
    const int c = 8 * lane;
    float ov[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, gv[8], wv[8];
    float ss = 0.f;
    if (c < v_dim) {
      load8_as_float(o + c, ov);
      load8_as_float(g + c, gv);
      load8_as_float(w + head * v_dim + c, wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += ov[j] * ov[j];
    }
    const float inv = rsqrtf(wave_sum(ss) / (float)v_dim + eps);
    if (c < v_dim) {
#pragma unroll
      for (int j = 0; j < 8; ++j) ov[j] = ov[j] * inv * wv[j] / (1.f + expf(-gv[j]));
      store8_from_float(dst + c, ov);
    }
    return;
  }
  float ss = 0.f;
  for (int c = lane; c < v_dim; c += WAVE) ss += o[c] * o[c];
  const float inv = rsqrtf(wave_sum(ss) / (float)v_dim + eps);
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
  const int vec = v_dim % 8 == 0 && v_dim <= 8 * WAVE && g_col % 8 == 0 && proj_stride % 8 == 0 &&
                  (((uintptr_t)o_raw | (uintptr_t)proj | (uintptr_t)w | (uintptr_t)out) & 15) == 0;
  if (is_f32)
    hipLaunchKernelGGL(mlstm_out_kernel<float>, grid, block, 0, stream, o_raw, (const float*)proj, proj_stride, g_col,
                       w, row_slot, (float*)out, n_heads, v_dim, eps, vec);
  else
    hipLaunchKernelGGL(mlstm_out_kernel<bf16_t>, grid, block, 0, stream, o_raw, (const bf16_t*)proj, proj_stride,
                       g_col, w, row_slot, (bf16_t*)out, n_heads, v_dim, eps, vec);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The same recurrence for steps of many rows in bfloat16, a chunk of 64 tokens at a time on the matrix cores.
// The running maximum obeys m_t = b_t + M_t with b_t the sum of the chunk's log forget gates up to t and
// M_t = max(m_0, max_(s<=t) c_s), c_s = i_s - b_s, so every weight of the chunk is known before any product:
//
//   o_t   = [ e_t (q_t . S_0) + sum_(s<=t) P_ts v_s ] / (max(|e_t (q_t . n_0) + sum_(s<=t) P_ts|, exp(-m_t)) + 1e-6)
//   P_ts  = (q_t . k_s) exp(c_s - M_t),   e_t = exp(m_0 - M_t)                       (both at most 1)
//   S_L   = exp(m_0 - M_L) S_0 + sum_s exp(c_s - M_L) k_s v_s^T,   n_L likewise,   m_L = b_L + M_L
//
// which is the token-by-token recurrence written out (same m_t, same weights). Gates, weights, maxima,
// normalisers, the decay of the state and the state itself are float32; the operands of the four products
// (q k^T, P v, q S_0, k^T v) are bfloat16 with float32 accumulation, as in attention. A workgroup of four waves
// owns one (sequence, head, 64 value columns) and walks the sequence's chunks in order with S^T in its
// accumulators: C[m = value column][n = key feature]. Operand layout of the 16x16x32 instruction as everywhere in
// this library: A lane (c, g) holds row c, k = 8g..8g+7; B likewise for column c; C lane holds rows 4g..4g+3 of
// column c. Products are arranged so that tokens (or key features) are the n index and operands come row-wise
// from LDS: scores^T = K Q^T, O^T = V^T P^T + S_0^T Q^T, dS^T = V^T K'. V^T and K'^T = (w_s k_s)^T are staged with the
// chunk's positions in the order in which the scores leave them in a lane (value_column).
#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16((a), (b), (c), 0, 0, 0)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define CH_L 64                 // tokens a chunk
#define CH_VS 64                // value columns a workgroup
#define CH_PAD 8
#define CH_MAX_DT 4             // tiles of 16 key features a wave may own: D <= 256

// Long prompts are also cut into segments of several chunks that run side by side, in three launches. MODE 1 of
// this kernel walks every segment but a sequence's last from an empty memory and leaves what the segment makes of
// one: (S, n, m) and the sum B of its log forget gates. Applying such a summary to a state (S_0, n_0, m_0) is
// m' = max(m_0 + B, m), S' = exp(m_0 + B - m') S_0 + exp(m - m') S. `mlstm_carry_kernel` does that from segment to
// segment, starting from the state the step found, and leaves the state that enters each segment (the S part in the
// summary's place). MODE 2 walks each segment from the state that enters it, as MODE 0 (one workgroup a sequence, no
// segments) walks a whole sequence; a sequence's last segment leaves the state, which no other workgroup of that
// launch reads. `tile_cu`: prefix sums over the sequences of their segments.
struct Segments {
  const int* tile_cu;
  int n_seqs, seg_rows;
  float *sum_s, *sum_n, *sum_m;       // [segments, heads, ...] as the state, and (m, B); sum_s becomes the entering S
  float *carry_n, *carry_m;           // [segments, heads, ...]: the n and m that enter each segment
};

template <int KB, int MODE>     // KB = ceil(D / 32)
__global__ __launch_bounds__(256) void mlstm_chunks_kernel(
    const bf16_t* __restrict__ proj, int64_t proj_stride, int q_col, int k_col, int v_col,
    const float* __restrict__ gates, const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state_s, float* __restrict__ state_n, float* __restrict__ state_m,
    float* __restrict__ o_raw, int n_heads, int dim, int v_dim, float q_scale, int write_state, Segments sg) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  constexpr int DP = 32 * KB;                                   // key features, padded with zeros
  constexpr int KS = DP + CH_PAD, TS = CH_L + CH_PAD;           // row strides in LDS
  constexpr int DT = (DP / 16 + 3) / 4;                         // key-feature tiles a wave owns
  const int head = blockIdx.y, v0 = blockIdx.z * CH_VS;
  int seq = blockIdx.x, seg = 0, seg_first = 0, n_segs = 1;
  if (MODE != 0) {                                              // blockIdx.x counts segments over all sequences
    if ((int)blockIdx.x >= sg.tile_cu[sg.n_seqs]) return;
    int lo = 0, hi = sg.n_seqs;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (sg.tile_cu[mid] <= (int)blockIdx.x) lo = mid; else hi = mid;
    }
    while (lo + 1 < sg.n_seqs && sg.tile_cu[lo + 1] <= (int)blockIdx.x) ++lo;
    seq = lo;
    seg_first = sg.tile_cu[seq];
    seg = blockIdx.x - seg_first;
    n_segs = sg.tile_cu[seq + 1] - seg_first;
  }
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int row0 = cu_rows[seq], n_tok = q_len[seq];
  const int tok_first = MODE == 0 ? 0 : seg * sg.seg_rows;
  const int tok_end = MODE == 0 ? n_tok : min(n_tok, tok_first + sg.seg_rows);
  const bool last_seg = seg == n_segs - 1;
  if (MODE == 1 && last_seg) return;                            // nobody folds a sequence's last segment
  bf16_t* k_s = (bf16_t*)lds_raw;                               // [64][KS]      keys, row-wise
  bf16_t* kw_t = k_s + CH_L * KS;                               // [DP][TS]      (w_s k_s)^T, positions permuted
  bf16_t* v_t = kw_t + DP * TS;                                 // [64][TS]      V^T, positions permuted
  bf16_t* s_t = v_t + CH_VS * TS;                               // [64][KS]      S_0^T rounded
  float* n_s = (float*)(s_t + CH_VS * KS);                      // [DP]
  float* g_M = n_s + DP;                                        // [64] M_t
  float* g_c = g_M + CH_L;                                      // [64] c_s
  float* g_b = g_c + CH_L;                                      // [64] b_t
  float* g_w = g_b + CH_L;                                      // [64] w_s = exp(c_s - M_L)
  float* g_x = g_w + CH_L;                                      // [4]  M_L, b_L
  const int64_t sh = (int64_t)slot * n_heads + head;
  float* S = state_s + sh * dim * v_dim;
  float* N = state_n + (sh * gridDim.z + blockIdx.z) * dim;     // n and m: this run of value columns' own copy
  float* M_state = state_m + sh * gridDim.z + blockIdx.z;
  const int64_t per_s = (int64_t)dim * v_dim;
  // where this workgroup's memory comes from: the state (a sequence of one segment reads the state itself in MODE 2
  // too: the workgroup that reads it is the one that writes it); nothing in MODE 1; in MODE 2 what the carry left
  const float* src_s = S;
  const float* src_n = N;
  const float* src_m = M_state;
  if (MODE == 2 && n_segs > 1) {
    const int64_t at = (int64_t)blockIdx.x * n_heads + head;
    src_s = sg.sum_s + at * per_s;
    src_n = sg.carry_n + at * dim;
    src_m = sg.carry_m + at;
  }
  const bool empty = MODE == 1;
  // the state: S^T tiles [value tile vt][own key-feature tile j], d-tile index = wave + 4 j
  f32x4 acc_s[4][DT];
#pragma unroll
  for (int vt = 0; vt < 4; ++vt)
#pragma unroll
    for (int j = 0; j < DT; ++j) {
      const int d = 16 * (wave + 4 * j) + c;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int v = v0 + 16 * vt + 4 * g + i;
        acc_s[vt][j][i] = (!empty && d < dim && v < v_dim) ? src_s[(int64_t)d * v_dim + v] : 0.f;
      }
    }
  for (int d = threadIdx.x; d < DP; d += blockDim.x) n_s[d] = (!empty && d < dim) ? src_n[d] : 0.f;
  float m0 = empty ? -INFINITY : src_m[0];
  float b_sum = 0.f;
  for (int t0 = tok_first; t0 < tok_end; t0 += CH_L) {
    const int nt = min(CH_L, tok_end - t0);
    __syncthreads();                                            // the chunk before is done with every buffer
    // S_0^T rounded, for the read-out of this chunk
    if (MODE != 1)
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int j = 0; j < DT; ++j) {
        const int d = 16 * (wave + 4 * j) + c;
        if (d < DP) {
#pragma unroll
          for (int i = 0; i < 4; ++i) s_t[(16 * vt + 4 * g + i) * KS + d] = float_to_bf16(acc_s[vt][j][i]);
        }
      }
    // the chunk's gates: one lane a token
    if (wave == 0) {
      const bool live = lane < nt;
      const float* gp = gates + (int64_t)(row0 + t0 + (live ? lane : 0)) * 2 * n_heads;
      const float gi = cap * tanhf((gp[head] + bias_i[head]) / cap);
      float b = live ? log_sigmoid(cap * tanhf((gp[n_heads + head] + bias_f[head]) / cap)) : 0.f;
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {                      // inclusive sum over the lanes before
        const float up = __shfl_up(b, o, WAVE);
        if (lane >= o) b += up;
      }
      const float cs = live ? gi - b : -INFINITY;
      float M = fmaxf(cs, lane == 0 ? m0 : -INFINITY);
#pragma unroll
      for (int o = 1; o < WAVE; o <<= 1) {
        const float up = __shfl_up(M, o, WAVE);
        if (lane >= o) M = fmaxf(M, up);
      }
      g_M[lane] = M;
      g_c[lane] = cs;
      g_b[lane] = b;
      g_w[lane] = live ? expf(cs - __shfl(M, nt - 1, WAVE)) : 0.f;
      if (lane == nt - 1) { g_x[0] = M; g_x[1] = b; }
    }
    __syncthreads();
    const float M_L = g_x[0], b_L = g_x[1];
    // stage the chunk: K row-wise; (w_s k_s)^T and V^T with the positions in the lanes' order
    // (neighbouring threads take neighbouring positions of the same features: their 2-byte writes into the
    // transposed copies then fall into one row, not into rows that share banks)
    for (int e = threadIdx.x; e < CH_L * (DP / 8); e += blockDim.x) {
      const int s = e % CH_L, d = 8 * (e / CH_L);
      float kv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (s < nt && d < dim)                                    // dim is a multiple of 8 (the host checks)
        load8_as_float(proj + (int64_t)(row0 + t0 + s) * proj_stride + k_col + (int64_t)head * dim + d, kv);
      store8_from_float(k_s + s * KS + d, kv);
      const float w = g_w[s];
      const int col = value_column(s);
#pragma unroll
      for (int j = 0; j < 8; ++j) kw_t[(d + j) * TS + col] = float_to_bf16(w * kv[j]);
    }
    for (int e = threadIdx.x; e < CH_L * (CH_VS / 8); e += blockDim.x) {
      const int s = e % CH_L, v = 8 * (e / CH_L);
      float vv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (s < nt && v0 + v < v_dim)                             // v_dim is a multiple of 8
        load8_as_float(proj + (int64_t)(row0 + t0 + s) * proj_stride + v_col + (int64_t)head * v_dim + v0 + v, vv);
      const int col = value_column(s);
#pragma unroll
      for (int j = 0; j < 8; ++j) v_t[(v + j) * TS + col] = float_to_bf16(vv[j]);
    }
    if (MODE == 1) __syncthreads();                             // the chunk is staged
    if (MODE != 1) {
    // this wave's 16 tokens: the queries stay in registers
    const int t = 16 * wave + c;                                // the lane's token of the chunk
    const bool t_live = t < nt;
    bf16x8 q[KB];
    float qn = 0.f;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int d = 32 * kb + 8 * g;
      float qv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (t_live && d < dim)
        load8_as_float(proj + (int64_t)(row0 + t0 + t) * proj_stride + q_col + (int64_t)head * dim + d, qv);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        q[kb][j] = (__bf16)qv[j];
        qn += qv[j] * n_s[d + j];
      }
    }
    qn += __shfl_xor(qn, 16, WAVE);
    qn += __shfl_xor(qn, 32, WAVE);
    __syncthreads();                                            // the chunk is staged
    const float M_t = t_live ? g_M[t] : 0.f;
    const float e_t = t_live ? expf(m0 - M_t) * q_scale : 0.f;
    f32x4 acc_o[4];
    if (16 * wave < nt) {
      // q S_0
#pragma unroll
      for (int vt = 0; vt < 4; ++vt) {
        acc_o[vt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          acc_o[vt] = MFMA16(*(const bf16x8*)(s_t + (16 * vt + c) * KS + 32 * kb + 8 * g), q[kb], acc_o[vt]);
        acc_o[vt] *= e_t;
      }
      // the chunk's own tokens up to each row
      float row_sum = 0.f;
      bf16x8 p[2];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) p[h][j] = (__bf16)0.f;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        if (st > wave) continue;                                // positions after all of the wave's rows
        f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          sc = MFMA16(*(const bf16x8*)(k_s + (16 * st + c) * KS + 32 * kb + 8 * g), q[kb], sc);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int s = 16 * st + 4 * g + i;
          const float pw = (t_live && s <= t) ? sc[i] * q_scale * expf(g_c[s] - M_t) : 0.f;
          row_sum += pw;
          p[st / 2][4 * (st & 1) + i] = (__bf16)pw;
        }
      }
      row_sum += __shfl_xor(row_sum, 16, WAVE);
      row_sum += __shfl_xor(row_sum, 32, WAVE);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (32 * h > 16 * wave + 15) continue;                  // a block of positions after all of the wave's rows
#pragma unroll
        for (int vt = 0; vt < 4; ++vt)
          acc_o[vt] = MFMA16(*(const bf16x8*)(v_t + (16 * vt + c) * TS + 32 * h + 8 * g), p[h], acc_o[vt]);
      }
      if (t_live) {
        const float m_t = g_b[t] + M_t;
        const float den = fmaxf(fabsf(e_t * qn + row_sum), expf(-m_t)) + 1e-6f;
        float* o = o_raw + ((int64_t)(row0 + t0 + t) * n_heads + head) * v_dim + v0;
#pragma unroll
        for (int vt = 0; vt < 4; ++vt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int v = 16 * vt + 4 * g + i;
            if (v0 + v < v_dim) o[v] = acc_o[vt][i] / den;
          }
      }
    }
    }
    // the state after the chunk
    const float decay = expf(m0 - M_L);
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int j = 0; j < DT; ++j) {
        if (16 * (wave + 4 * j) >= DP) continue;
        acc_s[vt][j] *= decay;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          acc_s[vt][j] = MFMA16(*(const bf16x8*)(v_t + (16 * vt + c) * TS + 32 * h + 8 * g),
                                *(const bf16x8*)(kw_t + (16 * (wave + 4 * j) + c) * TS + 32 * h + 8 * g), acc_s[vt][j]);
      }
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
      float a = decay * n_s[d];
      for (int s = 0; s < nt; ++s) a += g_w[s] * bf16_to_float(k_s[s * KS + d]);
      n_s[d] = a;
    }
    m0 = b_L + M_L;
    b_sum += b_L;
  }
  if (MODE == 1) {                                              // what the segment makes of a memory
    const int64_t at = (int64_t)blockIdx.x * n_heads + head;
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int j = 0; j < DT; ++j) {
        const int d = 16 * (wave + 4 * j) + c;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int v = v0 + 16 * vt + 4 * g + i;
          if (d < dim && v < v_dim) sg.sum_s[at * per_s + (int64_t)d * v_dim + v] = acc_s[vt][j][i];
        }
      }
    if (blockIdx.z == 0) {
      __syncthreads();
      for (int d = threadIdx.x; d < dim; d += blockDim.x) sg.sum_n[at * dim + d] = n_s[d];
      if (threadIdx.x == 0) { sg.sum_m[2 * at] = m0; sg.sum_m[2 * at + 1] = b_sum; }
    }
    return;
  }
  if (!write_state || !last_seg) return;
#pragma unroll
  for (int vt = 0; vt < 4; ++vt)
#pragma unroll
    for (int j = 0; j < DT; ++j) {
      const int d = 16 * (wave + 4 * j) + c;
      if (d >= dim) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int v = v0 + 16 * vt + 4 * g + i;
        if (v < v_dim) S[(int64_t)d * v_dim + v] = acc_s[vt][j][i];
      }
    }
  __syncthreads();
  for (int d = threadIdx.x; d < dim; d += blockDim.x) N[d] = n_s[d];
  if (threadIdx.x == 0) M_state[0] = m0;
}

// From segment to segment: the state that enters each (see above). Grid (sequence, head, run of 64 value columns);
// a thread keeps its elements of the run's slice of S in registers across the segments.
#define CARRY_SPLIT 4            // workgroups that share a run's rows of S
#define CARRY_HELD 16            // dim * 64 / 256 / CARRY_SPLIT for dim up to 256
__global__ __launch_bounds__(256) void mlstm_carry_kernel(const int* __restrict__ seq_slot,
                                                          const float* __restrict__ state_s,
                                                          const float* __restrict__ state_n,
                                                          const float* __restrict__ state_m, int n_heads, int dim,
                                                          int v_dim, Segments sg) {
  const int seq = blockIdx.x, head = blockIdx.y, run = blockIdx.z / CARRY_SPLIT, quarter = blockIdx.z % CARRY_SPLIT;
  const int runs = gridDim.z / CARRY_SPLIT, v0 = run * CH_VS;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = sg.tile_cu[seq], n_segs = sg.tile_cu[seq + 1] - first;
  if (n_segs <= 1) return;
  const int64_t sh = (int64_t)slot * n_heads + head, per_s = (int64_t)dim * v_dim;
  const float* S = state_s + sh * per_s;
  const int lane_v = threadIdx.x % CH_VS, d0 = threadIdx.x / CH_VS;      // element i of the thread: row 4 (d0 + 4 i) + quarter
  const bool v_ok = v0 + lane_v < v_dim;
  const bool writes_nm = run == 0 && quarter == 0;
  float cur[CARRY_HELD];
#pragma unroll
  for (int i = 0; i < CARRY_HELD; ++i) {
    const int d = 4 * (d0 + 4 * i) + quarter;
    cur[i] = (d < dim && v_ok) ? S[(int64_t)d * v_dim + v0 + lane_v] : 0.f;
  }
  float n_cur = (int)threadIdx.x < dim ? state_n[(sh * runs + run) * dim + threadIdx.x] : 0.f;
  float m_cur = state_m[sh * runs + run];
  for (int j = 0; j < n_segs; ++j) {
    const int64_t at = (int64_t)(first + j) * n_heads + head;
    const bool more = j < n_segs - 1;                       // the last segment has no summary, and nothing after it
    float keep = 1.f, take = 0.f, m_new = m_cur;
    if (more) {
      const float mk = sg.sum_m[2 * at], bk = sg.sum_m[2 * at + 1];
      m_new = fmaxf(m_cur + bk, mk);
      keep = expf(m_cur + bk - m_new);
      take = expf(mk - m_new);
    }
    float* ss = sg.sum_s + at * per_s;
    float add[CARRY_HELD];
#pragma unroll
    for (int i = 0; i < CARRY_HELD; ++i) {                  // all of the summary's values asked for before any is overwritten
      const int d = 4 * (d0 + 4 * i) + quarter;
      add[i] = (more && d < dim && v_ok) ? ss[(int64_t)d * v_dim + v0 + lane_v] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < CARRY_HELD; ++i) {
      const int d = 4 * (d0 + 4 * i) + quarter;
      if (d < dim && v_ok) {
        ss[(int64_t)d * v_dim + v0 + lane_v] = cur[i];
        cur[i] = keep * cur[i] + take * add[i];
      }
    }
    if ((int)threadIdx.x < dim) {
      const float more_n = more ? sg.sum_n[at * dim + threadIdx.x] : 0.f;
      if (writes_nm) sg.carry_n[at * dim + threadIdx.x] = n_cur;
      n_cur = keep * n_cur + take * more_n;
    }
    if (writes_nm && threadIdx.x == 0) sg.carry_m[at] = m_cur;
    m_cur = m_new;
  }
}

// Does the chunked kernel take these sizes? (16-byte pieces of rows; key width up to 256.)
DRYFT_API int dryft_mlstm_chunks_takes(int dim, int v_dim, int q_col, int k_col, int v_col, int64_t proj_stride) {
  return dim > 0 && dim <= 64 * CH_MAX_DT && dim % 8 == 0 && v_dim % 8 == 0 && q_col % 8 == 0 && k_col % 8 == 0 &&
         v_col % 8 == 0 && proj_stride % 8 == 0;
}

// seg_rows == 0: one workgroup walks a whole sequence. Otherwise (a multiple of 64): sequences are cut into
// segments of that many rows, `tile_cu` holding the prefix sums of their counts and `max_tiles` a bound on their
// total, and `scratch` room for the summaries: max_tiles * heads * (dim * v_dim + 2 * dim + 3) floats.
DRYFT_API int dryft_mlstm_chunks(const void* proj, int64_t proj_stride, int q_col, int k_col, int v_col,
                                 const float* gates, const float* bias_i, const float* bias_f, float cap,
                                 const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs, float* state_s,
                                 float* state_n, float* state_m, float* o_raw, int n_heads, int dim, int v_dim,
                                 float q_scale, int write_state, int seg_rows, const int* tile_cu, int max_tiles,
                                 float* scratch, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (!dryft_mlstm_chunks_takes(dim, v_dim, q_col, k_col, v_col, proj_stride) || ((uintptr_t)proj & 15) || !(cap > 0.f))
    return -1;
  if (seg_rows < 0 || seg_rows % CH_L || (seg_rows > 0 && (tile_cu == nullptr || scratch == nullptr || max_tiles <= 0)))
    return -1;
  const int kb = (dim + 31) / 32, dp = 32 * kb;
  const size_t lds = (size_t)(2 * CH_L * (dp + CH_PAD) + dp * (CH_L + CH_PAD) + CH_VS * (CH_L + CH_PAD)) * 2 +
                     (size_t)(dp + 4 * CH_L + 4) * sizeof(float);
  Segments sg = {};
  if (seg_rows > 0) {
    const size_t per = (size_t)n_heads * dim * v_dim, per_n = (size_t)n_heads * dim, per_m = (size_t)n_heads;
    sg.tile_cu = tile_cu; sg.n_seqs = n_seqs; sg.seg_rows = seg_rows;
    sg.sum_s = scratch;
    sg.sum_n = sg.sum_s + max_tiles * per;
    sg.sum_m = sg.sum_n + max_tiles * per_n;
    sg.carry_n = sg.sum_m + max_tiles * per_m * 2;
    sg.carry_m = sg.carry_n + max_tiles * per_n;
  }
  const int vs = (v_dim + CH_VS - 1) / CH_VS;
#define MC1(KBV, MODEV, GRIDX)                                                                                        \
  {                                                                                                                  \
    auto kernel = mlstm_chunks_kernel<KBV, MODEV>;                                                                   \
    if (lds > 64 * 1024 &&                                                                                           \
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return -1;                                                                                                     \
    hipLaunchKernelGGL(kernel, dim3(GRIDX, n_heads, vs), dim3(256), lds, stream, (const bf16_t*)proj, proj_stride,   \
                       q_col, k_col, v_col, gates, bias_i, bias_f, cap, seq_slot, cu_rows, q_len, state_s, state_n,    \
                       state_m, o_raw, n_heads, dim, v_dim, q_scale, write_state, sg);                               \
  }
#define MC(KBV)                                                                                                      \
  if (seg_rows == 0) MC1(KBV, 0, n_seqs) else {                                                                      \
    MC1(KBV, 1, max_tiles)                                                                                           \
    hipLaunchKernelGGL(mlstm_carry_kernel, dim3(n_seqs, n_heads, vs * CARRY_SPLIT), dim3(256), 0, stream, seq_slot, state_s, \
                       state_n, state_m, n_heads, dim, v_dim, sg);                                                   \
    MC1(KBV, 2, max_tiles)                                                                                           \
  }
  switch (kb) {
    case 1: MC(1); break;
    case 2: MC(2); break;
    case 3: MC(3); break;
    case 4: MC(4); break;
    case 5: MC(5); break;
    case 6: MC(6); break;
    case 7: MC(7); break;
    case 8: MC(8); break;
    default: return -1;
  }
#undef MC
#undef MC1
  return DRYFT_LAUNCH_CHECK();
}
