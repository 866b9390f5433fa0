// A matrix state per head with a token-dependent decay (RWKV-style time mixing): the token shift, the decay, the
// recurrence token by token, and the read-out's norm and gate. Everything here is float arithmetic; T is the
// dtype of the projections around it.
#include "common.h"

#define WKV_MAX_DIM 256
#define WKV_BLENDS 5

// ---------------------------------------------------------------------------------------------------
// Token shift. With h' the row before (of the same sequence; the state `previous[slot]` for a sequence's first row
// of the step, which is zeros when the sequence starts), blend b is h + (h' - h) * mu[b], rounded once.
// out is [5, rows, width]. One workgroup a row.
template <typename T>
__global__ __launch_bounds__(256) void wkv_blend_kernel(const T* __restrict__ h, const float* __restrict__ previous,
                                                        const float* __restrict__ mu, const int* __restrict__ row_slot,
                                                        const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                                                        const int* __restrict__ seq_start, T* __restrict__ out, int rows,
                                                        int width) {
  const int64_t row = blockIdx.x;
  const int slot = row_slot[row];
  const bool first = slot < 0 || row_pos[row] == seq_start[row_seq[row]];
  const int64_t plane = (int64_t)rows * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float x = load_as_float(h + row * width + c);
    float p = 0.f;
    if (!first) p = load_as_float(h + (row - 1) * width + c);
    else if (slot >= 0) p = previous[(int64_t)slot * width + c];
    const float d = p - x;
#pragma unroll
    for (int b = 0; b < WKV_BLENDS; ++b) store_from_float(out + b * plane + row * width + c, x + d * mu[b * width + c]);
  }
}

DRYFT_API int dryft_wkv_blend(const void* h, const float* previous, const float* mu, const int* row_slot,
                              const int* row_seq, const int* row_pos, const int* seq_start, void* out, int rows,
                              int width, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (is_f32)
    hipLaunchKernelGGL(wkv_blend_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)h, previous, mu, row_slot,
                       row_seq, row_pos, seq_start, (float*)out, rows, width);
  else
    hipLaunchKernelGGL(wkv_blend_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)h, previous, mu,
                       row_slot, row_seq, row_pos, seq_start, (bf16_t*)out, rows, width);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The decay's logarithm: log w = -exp(W_up tanh(low) + bias), with `low` [rows, rank] the float accumulators of
// the first projection. R rows a workgroup share each weight row they read; a thread owns outputs n, n + 256, ...
template <typename W, int R>
__global__ __launch_bounds__(256) void wkv_decay_kernel(const float* __restrict__ low, const W* __restrict__ up,
                                                        const float* __restrict__ bias, float* __restrict__ log_w,
                                                        int rows, int n_out, int rank) {
  extern __shared__ float t_low[];           // [R][rank]
  const int64_t row0 = (int64_t)blockIdx.x * R;
  for (int i = threadIdx.x; i < R * rank; i += blockDim.x) {
    const int64_t row = row0 + i / rank;
    t_low[i] = row < rows ? tanhf(low[row * rank + i % rank]) : 0.f;
  }
  __syncthreads();
  for (int n = threadIdx.x; n < n_out; n += blockDim.x) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    const W* w = up + (int64_t)n * rank;
    for (int j = 0; j < rank; ++j) {
      const float wj = load_as_float(w + j);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += wj * t_low[r * rank + j];
    }
    const float b = bias[n];
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (row0 + r < rows) log_w[(row0 + r) * n_out + n] = -expf(acc[r] + b);
  }
}

DRYFT_API int dryft_wkv_decay(const float* low, const void* up, const float* bias, float* log_w, int rows, int n_out,
                              int rank, int up_is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (rank <= 0 || rank > 2048) return -1;
  if (rows >= 64) {
    const size_t lds = (size_t)8 * rank * sizeof(float);
    dim3 grid((rows + 7) / 8);
    if (up_is_f32)
      hipLaunchKernelGGL((wkv_decay_kernel<float, 8>), grid, dim3(256), lds, stream, low, (const float*)up, bias, log_w,
                         rows, n_out, rank);
    else
      hipLaunchKernelGGL((wkv_decay_kernel<bf16_t, 8>), grid, dim3(256), lds, stream, low, (const bf16_t*)up, bias, log_w,
                         rows, n_out, rank);
  } else {
    const size_t lds = (size_t)rank * sizeof(float);
    if (up_is_f32)
      hipLaunchKernelGGL((wkv_decay_kernel<float, 1>), dim3(rows), dim3(256), lds, stream, low, (const float*)up, bias,
                         log_w, rows, n_out, rank);
    else
      hipLaunchKernelGGL((wkv_decay_kernel<bf16_t, 1>), dim3(rows), dim3(256), lds, stream, low, (const bf16_t*)up, bias,
                         log_w, rows, n_out, rank);
  }
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The recurrence, token by token. A wave takes 16 value columns of one (sequence, head): lane (c, q) keeps a quarter
// of column c of the state S [dim, dim] in registers (key channels q DK/4 .. (q+1) DK/4 - 1). The waves of a
// workgroup (up to four: 64 columns) share r, k, w = exp(log w) and the bonus u of eight tokens at a time through
// LDS. Per token
//
//   o_j = sum_i r_i S_ij + v_j sum_i r_i u_i k_i ;   S_ij <- w_i S_ij + k_i v_j
//
// with the sums over a lane's quarter first and over the four quarters by two exchanges between lanes. The wave of
// head 0 and column 0 also keeps the sequence's last input row as the next step's h' (`previous`), after every row
// of the step has been blended by the launch before.
#define WKV_GROUP 8

template <typename T, int DK>
__global__ __launch_bounds__(256) void wkv_steps_kernel(const T* __restrict__ r, const T* __restrict__ k,
                                                        const T* __restrict__ v, const float* __restrict__ log_w,
                                                        const float* __restrict__ bonus, const int* __restrict__ seq_slot,
                                                        const int* __restrict__ cu_rows, const int* __restrict__ q_len,
                                                        float* __restrict__ state, float* __restrict__ o_raw,
                                                        const T* __restrict__ h, float* __restrict__ previous, int hidden,
                                                        int n_heads, int dim, int write_state) {
  constexpr int DQ = DK / 4;
  __shared__ __attribute__((aligned(16))) float sh_r[WKV_GROUP][DK], sh_k[WKV_GROUP][DK], sh_w[WKV_GROUP][DK], sh_u[DK];
  const int seq = blockIdx.x, head = blockIdx.y;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, q = lane / 16;
  const int col = (blockIdx.z * (blockDim.x / WAVE) + wave) * 16 + c;
  const int slot = seq_slot[seq], row0 = cu_rows[seq], n = q_len[seq];
  const int inner = n_heads * dim;
  const bool owns = col < dim;
  if (slot < 0) {                      // a sequence that sits out: its rows of the output hold zeros
    for (int t = 0; t < n; ++t)
      if (owns && q == 0) o_raw[(int64_t)(row0 + t) * inner + head * dim + col] = 0.f;
    return;
  }
  if (n <= 0) return;
  float S[DQ];
  float* s_col = state + (((int64_t)slot * n_heads + head) * dim + q * DQ) * dim + col;
#pragma unroll
  for (int i = 0; i < DQ; ++i) S[i] = (owns && q * DQ + i < dim) ? s_col[(int64_t)i * dim] : 0.f;
  for (int i = threadIdx.x; i < DK; i += blockDim.x) sh_u[i] = i < dim ? bonus[head * dim + i] : 0.f;
  for (int t0 = 0; t0 < n; t0 += WKV_GROUP) {
    const int g = min(WKV_GROUP, n - t0);
    __syncthreads();
    for (int e = threadIdx.x; e < g * DK; e += blockDim.x) {
      const int t = e / DK, i = e % DK;
      const int64_t at = (int64_t)(row0 + t0 + t) * inner + head * dim + i;
      const bool in = i < dim;
      sh_r[t][i] = in ? load_as_float(r + at) : 0.f;
      sh_k[t][i] = in ? load_as_float(k + at) : 0.f;
      sh_w[t][i] = in ? expf(log_w[at]) : 0.f;
    }
    float vj[WKV_GROUP];
#pragma unroll
    for (int t = 0; t < WKV_GROUP; ++t)
      vj[t] = (owns && t < g) ? load_as_float(v + (int64_t)(row0 + t0 + t) * inner + head * dim + col) : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < WKV_GROUP; ++t) {
      if (t >= g) break;
      float o = 0.f, ruk = 0.f;
#pragma unroll
      for (int i = 0; i < DQ; i += 4) {
        const vf4 r4 = *(const vf4*)&sh_r[t][q * DQ + i], k4 = *(const vf4*)&sh_k[t][q * DQ + i];
        const vf4 w4 = *(const vf4*)&sh_w[t][q * DQ + i], u4 = *(const vf4*)&sh_u[q * DQ + i];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o += r4[e] * S[i + e];
          ruk += r4[e] * u4[e] * k4[e];
          S[i + e] = w4[e] * S[i + e] + k4[e] * vj[t];
        }
      }
      o += vj[t] * ruk;
      o += __shfl_xor(o, 16, WAVE);
      o += __shfl_xor(o, 32, WAVE);
      if (owns && q == 0) o_raw[(int64_t)(row0 + t0 + t) * inner + head * dim + col] = o;
    }
  }
  if (!write_state) return;
#pragma unroll
  for (int i = 0; i < DQ; ++i)
    if (owns && q * DQ + i < dim) s_col[(int64_t)i * dim] = S[i];
  if (head == 0 && blockIdx.z == 0 && wave == 0) {
    const T* last = h + (int64_t)(row0 + n - 1) * hidden;
    for (int cc = lane; cc < hidden; cc += WAVE) previous[(int64_t)slot * hidden + cc] = load_as_float(last + cc);
  }
}

template <typename T>
static int launch_wkv_steps(hipStream_t stream, const void* r, const void* k, const void* v, const float* log_w,
                            const float* bonus, const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs,
                            float* state, float* o_raw, const void* h, float* previous, int hidden, int n_heads, int dim,
                            int write_state) {
  const int waves = min(4, (dim + 15) / 16);                   // 16 value columns a wave
  dim3 grid(n_seqs, n_heads, (dim + 16 * waves - 1) / (16 * waves)), block(WAVE * waves);
#define WKV_CASE(DK)                                                                                               \
  hipLaunchKernelGGL((wkv_steps_kernel<T, DK>), grid, block, 0, stream, (const T*)r, (const T*)k, (const T*)v, log_w, \
                     bonus, seq_slot, cu_rows, q_len, state, o_raw, (const T*)h, previous, hidden, n_heads, dim,     \
                     write_state)
  if (dim <= 16) WKV_CASE(16);
  else if (dim <= 32) WKV_CASE(32);
  else if (dim <= 64) WKV_CASE(64);
  else if (dim <= 128) WKV_CASE(128);
  else WKV_CASE(256);
#undef WKV_CASE
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_wkv_max_dim() { return WKV_MAX_DIM; }

DRYFT_API int dryft_wkv_steps(const void* r, const void* k, const void* v, const float* log_w, const float* bonus,
                              const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs, float* state,
                              float* o_raw, const void* h, float* previous, int hidden, int n_heads, int dim,
                              int write_state, int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (dim <= 0 || dim > WKV_MAX_DIM || n_heads <= 0 || n_heads > 65535) return -1;
  if (is_f32)
    return launch_wkv_steps<float>(stream, r, k, v, log_w, bonus, seq_slot, cu_rows, q_len, n_seqs, state, o_raw, h,
                                   previous, hidden, n_heads, dim, write_state);
  return launch_wkv_steps<bf16_t>(stream, r, k, v, log_w, bonus, seq_slot, cu_rows, q_len, n_seqs, state, o_raw, h,
                                  previous, hidden, n_heads, dim, write_state);
}

// ---------------------------------------------------------------------------------------------------
// Read-out: out = o / sqrt(mean_head(o^2) + eps) * weight * silu(gate), one wave per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void wkv_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate,
                                                      const float* __restrict__ weight, T* __restrict__ out, int rows,
                                                      int n_heads, int dim, float eps) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t job = (int64_t)blockIdx.x * 4 + wave;
  if (job >= (int64_t)rows * n_heads) return;
  const int head = job % n_heads;
  const int64_t at = job * dim;
  float ss = 0.f;
  for (int i = lane; i < dim; i += WAVE) { const float o = o_raw[at + i]; ss += o * o; }
  ss = wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)dim + eps);
  for (int i = lane; i < dim; i += WAVE) {
    const float g = load_as_float(gate + at + i);
    store_from_float(out + at + i, o_raw[at + i] * rinv * weight[head * dim + i] * (g / (1.f + expf(-g))));
  }
}

DRYFT_API int dryft_wkv_out(const float* o_raw, const void* gate, const float* weight, void* out, int rows, int n_heads,
                            int dim, float eps, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  const int64_t jobs = (int64_t)rows * n_heads;
  dim3 grid((unsigned)((jobs + 3) / 4)), block(256);
  if (is_f32)
    hipLaunchKernelGGL(wkv_out_kernel<float>, grid, block, 0, stream, o_raw, (const float*)gate, weight, (float*)out, rows,
                       n_heads, dim, eps);
  else
    hipLaunchKernelGGL(wkv_out_kernel<bf16_t>, grid, block, 0, stream, o_raw, (const bf16_t*)gate, weight, (bf16_t*)out,
                       rows, n_heads, dim, eps);
  return DRYFT_LAUNCH_CHECK();
}
