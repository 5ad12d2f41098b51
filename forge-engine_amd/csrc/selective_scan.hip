// A selective state-space recurrence (Mamba) over a mixed batch, and the short causal convolution
// with its activation that feeds it.
//
//   fe_causal_conv_act:  y_t[c] = act(b[c] + sum_j w[c][j] * u_(t - taps + 1 + j)[c]), rows before the
//                        step from the sequence's state slot (its last taps - 1 rows of u, float32),
//                        rows before the sequence's start zeros (a slot is cleared when a request
//                        begins).  The state is moved on afterwards by fe_conv_state_update.
//   fe_selective_scan:   per sequence, channel c and state n, token after token,
//                          dt   = softplus(dt_lin[t][c] + dt_bias[c])
//                          S[c][n] <- exp(dt * A[c][n]) * S[c][n] + dt * x[t][c] * B[t][n]
//                          y[t][c] = (sum_n S[c][n] * C[t][n] + D[c] * x[t][c]) * silu(z[t][c])
//                        S lives in the sequence's state slot (float32) and is read at the start of the
//                        step and written at its end, so a sequence may be cut into steps anywhere.
//
// The scan: a block takes 256 / NS channels of one sequence; NS lanes share a channel and hold R of
// its states each in registers for the whole walk.  A chunk of 16 tokens is staged through LDS by the
// whole block (step sizes with their softplus applied once, x, z, and the B and C rows that every
// channel shares), walked, and its outputs stored together.  Everything between the loads and the
// stores is float32; exponentials are the accurate ones.
#include "common.h"

#define SS_THREADS 256
#define SS_CHUNK 16

template <typename T>
__global__ __launch_bounds__(SS_THREADS) void causal_conv_act_kernel(
    const T* __restrict__ u, size_t u_stride, const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ token_seq, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, T* __restrict__ out, int channels, int taps, int slots, int act) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * SS_THREADS + threadIdx.x;
  if (c >= channels) return;
  const int seq = token_seq[t];
  const int begin = cu_q[seq];
  const int slot = taps > 1 ? min(max(state_slots[seq], 0), slots - 1) : 0;
  const float* kept = taps > 1 ? state + (size_t)slot * (taps - 1) * channels : nullptr;
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int row = t - (taps - 1) + j;          // a row of this step, or of the state if before `begin`
    const float v = row >= begin ? load_as_float(u + (size_t)row * u_stride + c)
                                 : kept[(size_t)(taps - 1 - (begin - row)) * channels + c];
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  if (bias) acc += bias[c];
  if (act == 1) acc = acc / (1.f + expf(-acc));
  store_from_float(out + (size_t)t * channels + c, acc);
}

// u [T, >= channels] with row stride u_stride; w float32 [channels, taps] (the last column weighs the token
// itself); bias float32 [channels] or null; state float32 [slots, taps - 1, channels] (null for one tap);
// out [T, channels] dense.  act: 0 none, 1 silu.
extern "C" int fe_causal_conv_act(const void* u, int dtype, long long u_stride, const float* w, const float* bias,
                                  const float* state, const int* token_seq, const int* cu_q, const int* state_slots,
                                  void* out, int tokens, int channels, int taps, int slots, int act, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (channels <= 0 || taps < 1 || taps > 8 || u_stride < channels || !w || act < 0 || act > 1) return FE_BAD_ARGUMENT;
  if (taps > 1 && (!state || slots < 1)) return FE_BAD_ARGUMENT;
  const int channel_blocks = (channels + SS_THREADS - 1) / SS_THREADS;
  if (channel_blocks > 65535) return FE_BAD_ARGUMENT;
  const dim3 grid(tokens, channel_blocks);
  if (dtype == FE_F32)
    causal_conv_act_kernel<float><<<grid, SS_THREADS, 0, stream>>>((const float*)u, (size_t)u_stride, w, bias, state, token_seq,
                                                                   cu_q, state_slots, (float*)out, channels, taps, slots, act);
  else if (dtype == FE_BF16)
    causal_conv_act_kernel<bf16_t><<<grid, SS_THREADS, 0, stream>>>((const bf16_t*)u, (size_t)u_stride, w, bias, state, token_seq,
                                                                    cu_q, state_slots, (bf16_t*)out, channels, taps, slots, act);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

__device__ __forceinline__ float softplus_f32(float v) { return v > 20.f ? v : log1pf(expf(v)); }

template <typename T, int NS, int R>
__global__ __launch_bounds__(SS_THREADS) void selective_scan_kernel(
    const T* __restrict__ x, const float* __restrict__ dt_lin, const float* __restrict__ dt_bias,
    const float* __restrict__ A, const float* __restrict__ bc, size_t bc_stride, const float* __restrict__ D,
    const T* __restrict__ z, size_t z_stride, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, T* __restrict__ out, int C, int N, int slots, int tokens) {
  constexpr int CH = SS_THREADS / NS;
  __shared__ float s_dt[SS_CHUNK][CH], s_x[SS_CHUNK][CH], s_z[SS_CHUNK][CH], s_y[SS_CHUNK][CH];
  extern __shared__ float s_bc[];            // [SS_CHUNK][2 N]: a token's B row, then its C row
  const int seq = blockIdx.y;
  const int begin = cu_q[seq], end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (end <= begin || end > tokens || slot < 0 || slot >= slots) return;     // an empty (padding) sequence
  const int tid = threadIdx.x, cl = tid / NS, part = tid % NS;
  const int c0 = blockIdx.x * CH;
  const int c = c0 + cl;
  const bool c_ok = c < C;
  float s[R], a[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = part * R + i;
    const bool ok = c_ok && n < N;
    s[i] = ok ? state[((size_t)slot * C + c) * N + n] : 0.f;
    a[i] = ok ? A[(size_t)c * N + n] : 0.f;
  }
  const float d_c = c_ok ? D[c] : 0.f;
  const int two_n = 2 * N;

  for (int t0 = begin; t0 < end; t0 += SS_CHUNK) {
    const int len = min(SS_CHUNK, end - t0);
    __syncthreads();                         // the chunk before is consumed and its outputs are stored
    for (int e = tid; e < len * CH; e += SS_THREADS) {
      const int tt = e / CH, cc = e - tt * CH;
      const int gc = c0 + cc;
      if (gc < C) {
        const size_t at = (size_t)(t0 + tt) * C + gc;
        s_dt[tt][cc] = softplus_f32(dt_lin[at] + dt_bias[gc]);
        s_x[tt][cc] = load_as_float(x + at);
        s_z[tt][cc] = load_as_float(z + (size_t)(t0 + tt) * z_stride + gc);
      }
    }
    for (int e = tid; e < len * two_n; e += SS_THREADS) {
      const int tt = e / two_n, j = e - tt * two_n;
      s_bc[e] = bc[(size_t)(t0 + tt) * bc_stride + j];
    }
    __syncthreads();
    for (int tt = 0; tt < len; ++tt) {
      const float dtv = s_dt[tt][cl], xv = s_x[tt][cl];
      const float dx = dtv * xv;
      const float* brow = s_bc + tt * two_n;
      const float* crow = brow + N;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int n = part * R + i;
        if (n < N) {
          s[i] = fmaf(expf(dtv * a[i]), s[i], dx * brow[n]);
          acc = fmaf(s[i], crow[n], acc);
        }
      }
#pragma unroll
      for (int offset = NS / 2; offset > 0; offset >>= 1) acc += __shfl_xor(acc, offset, FE_WAVE);
      if (part == 0) {
        const float zv = s_z[tt][cl];
        s_y[tt][cl] = (acc + d_c * xv) * (zv / (1.f + expf(-zv)));
      }
    }
    __syncthreads();
    for (int e = tid; e < len * CH; e += SS_THREADS) {
      const int tt = e / CH, cc = e - tt * CH;
      if (c0 + cc < C) store_from_float(out + (size_t)(t0 + tt) * C + c0 + cc, s_y[tt][cc]);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = part * R + i;
    if (c_ok && n < N) state[((size_t)slot * C + c) * N + n] = s[i];
  }
}

// x [T, C] dense; dt_lin float32 [T, C] dense; dt_bias, D float32 [C]; A float32 [C, N] (negative: the decays'
// rates); bc float32 [T, >= 2 N] with row stride bc_stride (B, then C); z [T, >= C] with row stride z_stride;
// state float32 [slots, C, N]; out [T, C] dense.  lanes x per_lane >= N: lanes of a wave that share a channel
// (4, 8 or 16) and states each holds (4 with 4 or 8 lanes; 1, 2, 4, 8 or 16 with 16).
extern "C" int fe_selective_scan(const void* x, int dtype, const float* dt_lin, const float* dt_bias, const float* A,
                                 const float* bc, long long bc_stride, const float* D, const void* z, long long z_stride,
                                 float* state, const int* cu_q, const int* state_slots, void* out, int tokens, int num_seqs,
                                 int channels, int states, int slots, int lanes, int per_lane, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (channels <= 0 || states <= 0 || states > 256 || slots < 1 || bc_stride < 2LL * states || z_stride < channels ||
      lanes * per_lane < states || num_seqs > 65535)
    return FE_BAD_ARGUMENT;
  const size_t lds = (size_t)SS_CHUNK * 2 * states * sizeof(float);
  const dim3 grid((unsigned)(((long long)channels * lanes + SS_THREADS - 1) / SS_THREADS), num_seqs);
#define LAUNCH(T, NS, R)                                                                                          \
  selective_scan_kernel<T, NS, R><<<grid, SS_THREADS, lds, stream>>>(                                             \
      (const T*)x, dt_lin, dt_bias, A, bc, (size_t)bc_stride, D, (const T*)z, (size_t)z_stride, state, cu_q,      \
      state_slots, (T*)out, channels, states, slots, tokens)
#define SHAPES(T)                                                   \
  do {                                                              \
    if (lanes == 4 && per_lane == 4) LAUNCH(T, 4, 4);               \
    else if (lanes == 8 && per_lane == 4) LAUNCH(T, 8, 4);          \
    else if (lanes == 16 && per_lane == 1) LAUNCH(T, 16, 1);        \
    else if (lanes == 16 && per_lane == 2) LAUNCH(T, 16, 2);        \
    else if (lanes == 16 && per_lane == 4) LAUNCH(T, 16, 4);        \
    else if (lanes == 16 && per_lane == 8) LAUNCH(T, 16, 8);        \
    else if (lanes == 16 && per_lane == 16) LAUNCH(T, 16, 16);      \
    else return FE_BAD_ARGUMENT;                                    \
  } while (0)
  if (dtype == FE_F32) SHAPES(float);
  else if (dtype == FE_BF16) SHAPES(bf16_t);
  else return FE_BAD_ARGUMENT;
#undef SHAPES
#undef LAUNCH
  return fe_check_launch();
}
