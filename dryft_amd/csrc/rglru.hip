// A real-gated linear recurrent unit behind a short causal convolution (the recurrent block of Griffin),
// per sequence and channel. With x the recurrent branch's projection plus its bias, per channel c:
//
//   u_t = cb[c] + sum_j cw[c, j] x_(t - (taps - 1 - j))            (zeros before the sequence starts)
//   r = sigmoid(A_b u_b + ab),  i = sigmoid(I_b u_b + ib)          (u cut into equal blocks b, A_b and I_b square)
//   log a = -c_a * r * softplus(lam),  a = exp(log a)
//   S_t = a S_(t-1) + sqrt(1 - a^2) * i * u_t,     out_t = T( S_t * gelu_tanh(y_t + yb) )
//
// with y the other branch's projection. S and the last taps - 1 values of x live in float32 in the state
// store (zero when a sequence starts); everything above is float arithmetic and only out is rounded.
// Two kernels: the gates of every row at once (a workgroup takes a few rows of one block, so that each
// gate weight it reads serves all of them), then the walk over a sequence's rows, one thread a channel,
// which also leaves the state for the next step.
#include "common.h"

#define RG_ROWS 8               // rows a gates workgroup takes
#define RG_MAX_TAPS 16

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float soft_plus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// coef: float32 [rows, 2, width]: a, then sqrt(1 - a^2) * i * u.
template <typename T>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int x_col, const float* __restrict__ x_bias,
    const float* __restrict__ conv_w, const float* __restrict__ conv_b, int taps, const T* __restrict__ gate_a,
    const float* __restrict__ gate_a_bias, const T* __restrict__ gate_i, const float* __restrict__ gate_i_bias,
    const float* __restrict__ lam, float decay_scale, const int* __restrict__ row_slot,
    const int* __restrict__ row_seq, const int* __restrict__ row_pos, const int* __restrict__ seq_start,
    const float* __restrict__ tail, float* __restrict__ coef, int n_rows, int width, int block_size) {
  extern __shared__ float u_s[];                                // [RG_ROWS][block_size]
  const int r0 = blockIdx.x * RG_ROWS, b = blockIdx.y;
  const int rows = min(RG_ROWS, n_rows - r0);
  for (int e = threadIdx.x; e < rows * block_size; e += blockDim.x) {
    const int rr = e / block_size, c = e % block_size, ch = b * block_size + c;
    const int64_t row = r0 + rr;
    const int slot = row_slot[row];
    float u = 0.f;
    if (slot >= 0) {
      const int pos = row_pos[row], start = seq_start[row_seq[row]];
      u = conv_b[ch];
      for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j, p = pos - back;
        float x;
        if (p >= start) x = load_as_float(proj + (row - back) * proj_stride + x_col + ch) + x_bias[ch];
        else x = tail[((int64_t)slot * (taps - 1) + (taps - 1 - start + p)) * width + ch];   // zeros before the start
        u += conv_w[ch * taps + j] * x;
      }
    }
    u_s[e] = u;
  }
  __syncthreads();
  for (int o = threadIdx.x; o < block_size; o += blockDim.x) {
    const int ch = b * block_size + o;
    const T* wa = gate_a + ((int64_t)b * block_size + o) * block_size;
    const T* wi = gate_i + ((int64_t)b * block_size + o) * block_size;
    float acc_a[RG_ROWS], acc_i[RG_ROWS];
#pragma unroll
    for (int rr = 0; rr < RG_ROWS; ++rr) acc_a[rr] = acc_i[rr] = 0.f;
    for (int k = 0; k < block_size; ++k) {
      const float a = load_as_float(wa + k), i = load_as_float(wi + k);
#pragma unroll
      for (int rr = 0; rr < RG_ROWS; ++rr) {
        const float u = rr < rows ? u_s[rr * block_size + k] : 0.f;
        acc_a[rr] += a * u;
        acc_i[rr] += i * u;
      }
    }
    const float rate = decay_scale * soft_plus(lam[ch]);
#pragma unroll
    for (int rr = 0; rr < RG_ROWS; ++rr) {
      if (rr >= rows || row_slot[r0 + rr] < 0) continue;
      const float r = 1.f / (1.f + expf(-(acc_a[rr] + gate_a_bias[ch])));
      const float i = 1.f / (1.f + expf(-(acc_i[rr] + gate_i_bias[ch])));
      const float log_a = -rate * r;
      float* dst = coef + (int64_t)(r0 + rr) * 2 * width;
      dst[ch] = expf(log_a);
      dst[width + ch] = sqrtf(-expm1f(2.f * log_a)) * i * u_s[rr * block_size + o];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    const float* __restrict__ coef, const T* __restrict__ proj, int64_t proj_stride, int x_col, int y_col,
    const float* __restrict__ x_bias, const float* __restrict__ y_bias, int taps, const int* __restrict__ seq_slot,
    const int* __restrict__ cu_rows, const int* __restrict__ q_len, const int* __restrict__ row_slot,
    float* __restrict__ state, float* __restrict__ tail, T* __restrict__ out, int n_rows, int width, int write_state) {
  const int seq = blockIdx.x, ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= width) return;
  const int slot = seq_slot[seq];
  const int row0 = cu_rows[seq], n_tok = q_len[seq];
  if (slot < 0) {                                               // the rows of a sequence that sits out hold zeros
    for (int t = 0; t < n_tok; ++t) store_from_float(out + (int64_t)(row0 + t) * width + ch, 0.f);
    return;
  }
  float S = state[(int64_t)slot * width + ch];
  const float yb = y_bias[ch];
  for (int t = 0; t < n_tok; ++t) {
    const int64_t row = row0 + t;
    const float* c = coef + row * 2 * width;
    S = c[ch] * S + c[width + ch];
    const float y = gelu_tanh(load_as_float(proj + row * proj_stride + y_col + ch) + yb);
    store_from_float(out + row * width + ch, S * y);
  }
  if (!write_state) return;
  state[(int64_t)slot * width + ch] = S;
  // the convolution's memory: the last taps - 1 inputs of the sequence, oldest first
  const int keep = taps - 1;
  float old[RG_MAX_TAPS];
  float* tl = tail + (int64_t)slot * keep * width + ch;
  for (int j = 0; j < keep; ++j) old[j] = tl[(int64_t)j * width];
  for (int j = 0; j < keep; ++j) {
    const int t = n_tok - keep + j;                             // the step's token that lands in place j
    float v;
    if (t >= 0) v = load_as_float(proj + (int64_t)(row0 + t) * proj_stride + x_col + ch) + x_bias[ch];
    else v = old[j + n_tok];                                    // fewer new tokens than places: the old ones move up
    tl[(int64_t)j * width] = v;
  }
}

// ---------------------------------------------------------------------------------------------------
// The same walk for steps of many rows, cut into tiles of RG_TILE tokens so that a long prompt fills the chip.
// S_t = a_t S_(t-1) + b_t is linear in S, so a tile is summed up by two numbers per channel, P = prod a and
// Q = the tile's last S from S = 0. Three launches: every tile's (P, Q); per sequence and channel the state that
// enters each tile, S <- P S + Q from tile to tile (a few dozen steps; this one also leaves the state and the
// convolution's memory for the next step, and is the only one that touches them); every tile's own tokens from
// the state that enters it. `tile_cu` are the prefix sums over the sequences of their tiles (a sequence that
// sits out has none).
#define RG_TILE 64

__device__ __forceinline__ bool rg_locate(int tile, const int* __restrict__ tile_cu, int n_seqs, int& seq, int& in_seq) {
  if (tile >= tile_cu[n_seqs]) return false;
  int lo = 0, hi = n_seqs;                                      // last seq with tile_cu[seq] <= tile
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (tile_cu[mid] <= tile) lo = mid; else hi = mid;
  }
  while (lo + 1 < n_seqs && tile_cu[lo + 1] <= tile) ++lo;      // sequences without tiles share a start
  seq = lo;
  in_seq = tile - tile_cu[lo];
  return true;
}

// ends: float32 [tiles, 2, width]: P, then Q.
__global__ __launch_bounds__(256) void rglru_tile_ends_kernel(const float* __restrict__ coef,
                                                              const int* __restrict__ cu_rows,
                                                              const int* __restrict__ q_len,
                                                              const int* __restrict__ tile_cu, int n_seqs,
                                                              float* __restrict__ ends, int width) {
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  int seq, j;
  if (!rg_locate(blockIdx.x, tile_cu, n_seqs, seq, j) || ch >= width) return;
  const int t0 = j * RG_TILE, t1 = min(q_len[seq], t0 + RG_TILE);
  float P = 1.f, Q = 0.f;
  const float* c0 = coef + (int64_t)cu_rows[seq] * 2 * width + ch;
  int t = t0;
  for (; t + 8 <= t1; t += 8) {                                 // eight tokens' coefficients asked for together
    float a[8], bb[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) { a[u] = c0[(int64_t)(t + u) * 2 * width]; bb[u] = c0[(int64_t)(t + u) * 2 * width + width]; }
#pragma unroll
    for (int u = 0; u < 8; ++u) { P *= a[u]; Q = a[u] * Q + bb[u]; }
  }
  for (; t < t1; ++t) {
    const float a = c0[(int64_t)t * 2 * width], bb = c0[(int64_t)t * 2 * width + width];
    P *= a;
    Q = a * Q + bb;
  }
  ends[((int64_t)blockIdx.x * 2) * width + ch] = P;
  ends[((int64_t)blockIdx.x * 2 + 1) * width + ch] = Q;
}

// Turns ends[tile] = (P, Q) into ends[tile][0] = the state that enters the tile; leaves the step's last state.
template <typename T>
__global__ __launch_bounds__(256) void rglru_carry_kernel(
    float* __restrict__ ends, const T* __restrict__ proj, int64_t proj_stride, int x_col,
    const float* __restrict__ x_bias, int taps, const int* __restrict__ seq_slot, const int* __restrict__ cu_rows,
    const int* __restrict__ q_len, const int* __restrict__ tile_cu, float* __restrict__ state,
    float* __restrict__ tail, int width, int write_state) {
  const int seq = blockIdx.x, ch = blockIdx.y * blockDim.x + threadIdx.x;
  if (ch >= width) return;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int row0 = cu_rows[seq], n_tok = q_len[seq];
  float S = state[(int64_t)slot * width + ch];
  for (int k = tile_cu[seq]; k < tile_cu[seq + 1]; ++k) {
    float* e = ends + ((int64_t)k * 2) * width;
    const float P = e[ch], Q = e[width + ch];
    e[ch] = S;
    S = P * S + Q;
  }
  if (!write_state) return;
  state[(int64_t)slot * width + ch] = S;
  const int keep = taps - 1;
  float old[RG_MAX_TAPS];
  float* tl = tail + (int64_t)slot * keep * width + ch;
  for (int j = 0; j < keep; ++j) old[j] = tl[(int64_t)j * width];
  for (int j = 0; j < keep; ++j) {
    const int t = n_tok - keep + j;
    float v;
    if (t >= 0) v = load_as_float(proj + (int64_t)(row0 + t) * proj_stride + x_col + ch) + x_bias[ch];
    else v = old[j + n_tok];
    tl[(int64_t)j * width] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rglru_apply_tiles_kernel(
    const float* __restrict__ coef, const float* __restrict__ ends, const T* __restrict__ proj, int64_t proj_stride,
    int y_col, const float* __restrict__ y_bias, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    const int* __restrict__ tile_cu, int n_seqs, T* __restrict__ out, int width) {
  const int ch = blockIdx.y * blockDim.x + threadIdx.x;
  int seq, j;
  if (!rg_locate(blockIdx.x, tile_cu, n_seqs, seq, j) || ch >= width) return;
  float S = ends[((int64_t)blockIdx.x * 2) * width + ch];
  const float yb = y_bias[ch];
  const int t0 = j * RG_TILE, t1 = min(q_len[seq], t0 + RG_TILE);
  const int64_t first = cu_rows[seq];
  int t = t0;
  for (; t + 8 <= t1; t += 8) {                                 // eight tokens' operands asked for together
    float a[8], bb[8], y[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t row = first + t + u;
      a[u] = coef[row * 2 * width + ch];
      bb[u] = coef[row * 2 * width + width + ch];
      y[u] = load_as_float(proj + row * proj_stride + y_col + ch);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      S = a[u] * S + bb[u];
      store_from_float(out + (first + t + u) * width + ch, S * gelu_tanh(y[u] + yb));
    }
  }
  for (; t < t1; ++t) {
    const int64_t row = first + t;
    const float* c = coef + row * 2 * width;
    S = c[ch] * S + c[width + ch];
    const float y = gelu_tanh(load_as_float(proj + row * proj_stride + y_col + ch) + yb);
    store_from_float(out + row * width + ch, S * y);
  }
}

DRYFT_API int dryft_rglru_tile_rows() { return RG_TILE; }

// out must hold zeros (or anything finite) in the rows of sequences that sit out: no tile visits them.
DRYFT_API int dryft_rglru_scan_tiles(const float* coef, float* ends, const void* proj, int64_t proj_stride, int x_col,
                                     int y_col, const float* x_bias, const float* y_bias, int taps, const int* seq_slot,
                                     const int* cu_rows, const int* q_len, const int* tile_cu, int n_seqs,
                                     int max_tiles, float* state, float* tail, void* out, int width, int write_state,
                                     int is_f32, hipStream_t stream) {
  if (n_seqs <= 0 || max_tiles <= 0) return 0;
  if (taps < 1 || taps > RG_MAX_TAPS) return -1;
  const int cb = (width + 255) / 256;
  if (cb > 65535) return -1;
  hipLaunchKernelGGL(rglru_tile_ends_kernel, dim3(max_tiles, cb), dim3(256), 0, stream, coef, cu_rows, q_len, tile_cu,
                     n_seqs, ends, width);
  if (is_f32) {
    hipLaunchKernelGGL(rglru_carry_kernel<float>, dim3(n_seqs, cb), dim3(256), 0, stream, ends, (const float*)proj,
                       proj_stride, x_col, x_bias, taps, seq_slot, cu_rows, q_len, tile_cu, state, tail, width,
                       write_state);
    hipLaunchKernelGGL(rglru_apply_tiles_kernel<float>, dim3(max_tiles, cb), dim3(256), 0, stream, coef, ends,
                       (const float*)proj, proj_stride, y_col, y_bias, cu_rows, q_len, tile_cu, n_seqs, (float*)out,
                       width);
  } else {
    hipLaunchKernelGGL(rglru_carry_kernel<bf16_t>, dim3(n_seqs, cb), dim3(256), 0, stream, ends, (const bf16_t*)proj,
                       proj_stride, x_col, x_bias, taps, seq_slot, cu_rows, q_len, tile_cu, state, tail, width,
                       write_state);
    hipLaunchKernelGGL(rglru_apply_tiles_kernel<bf16_t>, dim3(max_tiles, cb), dim3(256), 0, stream, coef, ends,
                       (const bf16_t*)proj, proj_stride, y_col, y_bias, cu_rows, q_len, tile_cu, n_seqs, (bf16_t*)out,
                       width);
  }
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The gates on the matrix cores, for bfloat16 and blocks whose size is a multiple of 32. A workgroup takes up to
// 64 rows of one block: it forms their convolution in float into LDS, then every wave multiplies its 16 rows with
// the block's two gate matrices, 16 outputs at a time: C[m = output][n = row] = sum_k W[output][k] u[row][k], the
// weights straight from memory (16 bytes a lane along k), u rounded to bfloat16 on its way out of LDS, the sums
// float32. What follows the product (biases, sigmoids, the decay and its square root, the multiplication with the
// unrounded u) is float arithmetic on the accumulators. With at most 16 rows in the step (decoding) the four
// waves share those rows and deal the outputs among themselves, and among `gridDim.z` workgroups.
#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16((a), (b), (c), 0, 0, 0)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
#define RG_MM_ROWS 64
#define RG_MM_PAD 4

__global__ __launch_bounds__(256) void rglru_gates_mfma_kernel(
    const bf16_t* __restrict__ proj, int64_t proj_stride, int x_col, const float* __restrict__ x_bias,
    const float* __restrict__ conv_w, const float* __restrict__ conv_b, int taps, const bf16_t* __restrict__ gate_a,
    const float* __restrict__ gate_a_bias, const bf16_t* __restrict__ gate_i, const float* __restrict__ gate_i_bias,
    const float* __restrict__ lam, float decay_scale, const int* __restrict__ row_slot,
    const int* __restrict__ row_seq, const int* __restrict__ row_pos, const int* __restrict__ seq_start,
    const float* __restrict__ tail, float* __restrict__ coef, int n_rows, int width, int block_size, int few) {
  extern __shared__ __attribute__((aligned(16))) float u_s[];   // [rows of the workgroup][block_size + pad]
  const int wg_rows = few ? 16 : RG_MM_ROWS;
  const int r0 = blockIdx.x * wg_rows, b = blockIdx.y, ld = block_size + RG_MM_PAD;
  const int rows = min(wg_rows, n_rows - r0);
  // the rows' facts once; then a thread takes one channel and walks a run of the rows in order, so that the
  // convolution's window slides: a row that follows its predecessor in the same sequence brings one new input
  __shared__ int r_slot[RG_MM_ROWS], r_pos[RG_MM_ROWS], r_start[RG_MM_ROWS];
  if (threadIdx.x < wg_rows) {
    int slot = -1, pos = 0, start = 0;
    if ((int)threadIdx.x < rows) {
      const int64_t row = r0 + threadIdx.x;
      slot = row_slot[row];
      if (slot >= 0) { pos = row_pos[row]; start = seq_start[row_seq[row]]; }
    }
    r_slot[threadIdx.x] = slot; r_pos[threadIdx.x] = pos; r_start[threadIdx.x] = start;
  }
  __syncthreads();
  {
    const int ch_threads = min(block_size, (int)blockDim.x), groups = blockDim.x / ch_threads;
    const int grp = threadIdx.x / ch_threads, per = (wg_rows + groups - 1) / groups;
    const int rr0 = grp * per, rr1 = grp < groups ? min(wg_rows, rr0 + per) : 0;
    for (int cc = threadIdx.x % ch_threads; cc < block_size && rr0 < rr1; cc += ch_threads) {
      const int ch = b * block_size + cc;
      // taps and window sit at the end of arrays of fixed size (place k holds the input `15 - k` positions back)
      float cw[RG_MAX_TAPS], win[RG_MAX_TAPS];
#pragma unroll
      for (int k = 0; k < RG_MAX_TAPS; ++k) {
        cw[k] = k >= RG_MAX_TAPS - taps ? conv_w[ch * taps + k - (RG_MAX_TAPS - taps)] : 0.f;
        win[k] = 0.f;
      }
      const float xb = x_bias[ch], cb = conv_b[ch];
      for (int rr = rr0; rr < rr1; ++rr) {
        const int slot = r_slot[rr];
        float u = 0.f;
        if (slot >= 0) {
          const int pos = r_pos[rr], start = r_start[rr];
          const int64_t row = r0 + rr;
          const bool slides = rr > rr0 && r_slot[rr - 1] == slot && r_pos[rr - 1] == pos - 1;
          if (slides) {
#pragma unroll
            for (int k = 0; k < RG_MAX_TAPS - 1; ++k) win[k] = win[k + 1];
            win[RG_MAX_TAPS - 1] = load_as_float(proj + row * proj_stride + x_col + ch) + xb;
          } else {
#pragma unroll
            for (int k = 0; k < RG_MAX_TAPS; ++k) {
              if (k < RG_MAX_TAPS - taps) continue;
              const int back = RG_MAX_TAPS - 1 - k, p = pos - back;
              if (p >= start) win[k] = load_as_float(proj + (row - back) * proj_stride + x_col + ch) + xb;
              else win[k] = tail[((int64_t)slot * (taps - 1) + (taps - 1 - start + p)) * width + ch];  // zeros before the start
            }
          }
          u = cb;
#pragma unroll
          for (int k = 0; k < RG_MAX_TAPS; ++k) u += cw[k] * win[k];
        }
        u_s[rr * ld + cc] = u;
      }
    }
  }
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int row_tile = few ? 0 : wave;                           // the wave's 16 rows within the workgroup's
  if (16 * row_tile >= rows) return;
  const int tiles = block_size / 16, kbs = block_size / 32;
  const int first = few ? blockIdx.z * 4 + wave : 0, stride = few ? 4 * gridDim.z : 1;
  const float* u_row = u_s + (16 * row_tile + c) * ld;
  const int64_t row = r0 + 16 * row_tile + c;
  const bool live = 16 * row_tile + c < rows && row_slot[min(row, (int64_t)n_rows - 1)] >= 0;
  for (int ot = first; ot < tiles; ot += stride) {
    const bf16_t* wa = gate_a + ((int64_t)b * block_size + 16 * ot + c) * block_size + 8 * g;
    const bf16_t* wi = gate_i + ((int64_t)b * block_size + 16 * ot + c) * block_size + 8 * g;
    f32x4 acc_a = f32x4{0.f, 0.f, 0.f, 0.f}, acc_i = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; kb < kbs; ++kb) {
      const vf4 lo = *(const vf4*)(u_row + 32 * kb + 8 * g), hi = *(const vf4*)(u_row + 32 * kb + 8 * g + 4);
      bf16x8 ub;
#pragma unroll
      for (int j = 0; j < 4; ++j) { ub[j] = (__bf16)lo[j]; ub[4 + j] = (__bf16)hi[j]; }
      acc_a = MFMA16(*(const bf16x8*)(wa + 32 * kb), ub, acc_a);
      acc_i = MFMA16(*(const bf16x8*)(wi + 32 * kb), ub, acc_i);
    }
    if (!live) continue;
    const int o = 16 * ot + 4 * g, ch = b * block_size + o;      // the lane's four outputs of its row
    vf4 va, vb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float r = 1.f / (1.f + expf(-(acc_a[i] + gate_a_bias[ch + i])));
      const float gi = 1.f / (1.f + expf(-(acc_i[i] + gate_i_bias[ch + i])));
      const float log_a = -decay_scale * soft_plus(lam[ch + i]) * r;
      va[i] = expf(log_a);
      vb[i] = sqrtf(-expm1f(2.f * log_a)) * gi * u_row[o + i];
    }
    float* dst = coef + row * 2 * width + ch;
    *(vf4*)dst = va;
    *(vf4*)(dst + width) = vb;
  }
}

DRYFT_API int dryft_rglru_gates(const void* proj, int64_t proj_stride, int x_col, const float* x_bias,
                                const float* conv_w, const float* conv_b, int taps, const void* gate_a,
                                const float* gate_a_bias, const void* gate_i, const float* gate_i_bias,
                                const float* lam, float decay_scale, const int* row_slot, const int* row_seq,
                                const int* row_pos, const int* seq_start, const float* tail, float* coef, int n_rows,
                                int width, int blocks, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (blocks <= 0 || width % blocks || taps < 1 || taps > RG_MAX_TAPS) return -1;
  const int block_size = width / blocks;
  // bfloat16 blocks of a multiple of 32 channels go to the matrix cores (16-byte pieces of the weights' rows)
  const size_t mm_lds = (size_t)(n_rows <= 16 ? 16 : RG_MM_ROWS) * (block_size + RG_MM_PAD) * sizeof(float);
  if (!is_f32 && block_size % 32 == 0 && mm_lds <= 150 * 1024 && width % 4 == 0 &&
      (((uintptr_t)gate_a | (uintptr_t)gate_i | (uintptr_t)coef) & 15) == 0) {
    const int few = n_rows <= 16;
    const int tiles = block_size / 16;
    dim3 mgrid(few ? 1 : (n_rows + RG_MM_ROWS - 1) / RG_MM_ROWS, blocks, few ? min(4, (tiles + 3) / 4) : 1);
    if (mm_lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)rglru_gates_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)mm_lds) != hipSuccess)
      return -1;
    hipLaunchKernelGGL(rglru_gates_mfma_kernel, mgrid, dim3(256), mm_lds, stream, (const bf16_t*)proj, proj_stride,
                       x_col, x_bias, conv_w, conv_b, taps, (const bf16_t*)gate_a, gate_a_bias, (const bf16_t*)gate_i,
                       gate_i_bias, lam, decay_scale, row_slot, row_seq, row_pos, seq_start, tail, coef, n_rows, width,
                       block_size, few);
    return DRYFT_LAUNCH_CHECK();
  }
  const size_t lds = (size_t)RG_ROWS * block_size * sizeof(float);
  if (lds > 64 * 1024) return -1;
  dim3 grid((n_rows + RG_ROWS - 1) / RG_ROWS, blocks), block(256);
  if (is_f32)
    hipLaunchKernelGGL(rglru_gates_kernel<float>, grid, block, lds, stream, (const float*)proj, proj_stride, x_col,
                       x_bias, conv_w, conv_b, taps, (const float*)gate_a, gate_a_bias, (const float*)gate_i,
                       gate_i_bias, lam, decay_scale, row_slot, row_seq, row_pos, seq_start, tail, coef, n_rows, width,
                       block_size);
  else
    hipLaunchKernelGGL(rglru_gates_kernel<bf16_t>, grid, block, lds, stream, (const bf16_t*)proj, proj_stride, x_col,
                       x_bias, conv_w, conv_b, taps, (const bf16_t*)gate_a, gate_a_bias, (const bf16_t*)gate_i,
                       gate_i_bias, lam, decay_scale, row_slot, row_seq, row_pos, seq_start, tail, coef, n_rows, width,
                       block_size);
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_rglru_scan(const float* coef, const void* proj, int64_t proj_stride, int x_col, int y_col,
                               const float* x_bias, const float* y_bias, int taps, const int* seq_slot,
                               const int* cu_rows, const int* q_len, const int* row_slot, int n_seqs, float* state,
                               float* tail, void* out, int n_rows, int width, int write_state, int is_f32,
                               hipStream_t stream) {
  if (n_seqs <= 0 || n_rows <= 0) return 0;
  if (taps < 1 || taps > RG_MAX_TAPS) return -1;
  dim3 grid(n_seqs, (width + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(rglru_scan_kernel<float>, grid, block, 0, stream, coef, (const float*)proj, proj_stride, x_col,
                       y_col, x_bias, y_bias, taps, seq_slot, cu_rows, q_len, row_slot, state, tail, (float*)out,
                       n_rows, width, write_state);
  else
    hipLaunchKernelGGL(rglru_scan_kernel<bf16_t>, grid, block, 0, stream, coef, (const bf16_t*)proj, proj_stride,
                       x_col, y_col, x_bias, y_bias, taps, seq_slot, cu_rows, q_len, row_slot, state, tail,
                       (bf16_t*)out, n_rows, width, write_state);
  return DRYFT_LAUNCH_CHECK();
}
