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
// whole block (step sizes with their softplus applied once, x, and the B and C rows that every channel
// shares), walked, and its outputs (with the skip's term and the gate) stored together.  Everything
// between the loads and the stores is float32.  A decay is 2^(dt A log2 e) by the hardware's power of
// two: its argument is never positive, its error is about one unit in the last place, and the rounding
// of the argument weighs least where the decay is near one.
// A long step of one sequence is cut into segments that are walked side by side (see
// fe_selective_scan): the walk is serial in the tokens, and one block a channel group leaves most of
// the chip's wave slots empty.
#include "common.h"

#define SS_THREADS 256
#define SS_CHUNK 16

#define CONV_MAX_TAPS 8

// VEC neighbouring channels of one row as floats (one load of VEC elements when VEC > 1: the caller has
// checked the alignment).
template <typename T, int VEC>
__device__ __forceinline__ void load_channels(const T* p, float (&v)[VEC]) {
  struct alignas(sizeof(T) * VEC) Pack { T e[VEC]; };
  const Pack pack = *reinterpret_cast<const Pack*>(p);
#pragma unroll
  for (int i = 0; i < VEC; ++i) v[i] = load_as_float(&pack.e[i]);
}

template <typename T, int VEC>
__device__ __forceinline__ void store_channels(T* p, const float (&v)[VEC]) {
  struct alignas(sizeof(T) * VEC) Pack { T e[VEC]; };
  Pack pack;
#pragma unroll
  for (int i = 0; i < VEC; ++i) store_from_float(&pack.e[i], v[i]);
  *reinterpret_cast<Pack*>(p) = pack;
}

// A thread takes VEC neighbouring channels over a run of `run` rows of the step and keeps the rows that the
// taps reach in registers, so that a row of u is loaded once a run; a row before the sequence's part of
// the step comes from the sequence's state instead (rows of u are indexed by the step's rows whatever
// sequence they belong to, so the registers' rows are the right ones wherever the row is of this step).
template <typename T, int VEC>
__global__ __launch_bounds__(SS_THREADS) void causal_conv_act_kernel(
    const T* __restrict__ u, size_t u_stride, const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, const int* __restrict__ token_seq, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, T* __restrict__ out, int channels, int taps, int slots, int act, int tokens, int run) {
  const int t0 = blockIdx.x * run;
  const int c = (blockIdx.y * SS_THREADS + threadIdx.x) * VEC;
  if (c >= channels) return;
  float weight[CONV_MAX_TAPS][VEC], rows[CONV_MAX_TAPS][VEC], b[VEC];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      weight[j][i] = j < taps ? w[(size_t)(c + i) * taps + j] : 0.f;
      rows[j][i] = 0.f;
    }
  }
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    // rows[j] is the step's row t - (taps - 1) + j for the run's token t: ahead of the first, all but the last
    const int row = t0 - (taps - 1) + j;
    if (j + 1 < taps && row >= 0) load_channels<T, VEC>(u + (size_t)row * u_stride + c, rows[j + 1 < CONV_MAX_TAPS ? j + 1 : j]);
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) b[i] = bias ? bias[c + i] : 0.f;
  const int t_end = min(tokens, t0 + run);
  for (int t = t0; t < t_end; ++t) {
#pragma unroll
    for (int j = 0; j + 1 < CONV_MAX_TAPS; ++j) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) rows[j][i] = rows[j + 1][i];
    }
    // the newest row sits at index taps - 1; the shift above moved every older one down by one
    float newest[VEC];
    load_channels<T, VEC>(u + (size_t)t * u_stride + c, newest);
    const int seq = token_seq[t];
    const int begin = cu_q[seq];
    const int slot = taps > 1 ? min(max(state_slots[seq], 0), slots - 1) : 0;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = b[i];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
      if (j < taps) {
        if (j == taps - 1) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) rows[j][i] = newest[i];
        }
        const int row = t - (taps - 1) + j;
        if (row >= begin) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[i] = fmaf(weight[j][i], rows[j][i], acc[i]);
        } else {          // a row of the steps before: the state holds the last taps - 1 of them
          const float* kept = state + ((size_t)slot * (taps - 1) + (taps - 1 - (begin - row))) * channels + c;
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[i] = fmaf(weight[j][i], kept[i], acc[i]);
        }
      }
    }
    if (act == 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] = acc[i] / (1.f + expf(-acc[i]));
    }
    store_channels<T, VEC>(out + (size_t)t * channels + c, acc);
  }
}

// u [T, >= channels] with row stride u_stride; w float32 [channels, taps] (the last column weighs the token
// itself); bias float32 [channels] or null; state float32 [slots, taps - 1, channels] (null for one tap);
// out [T, channels] dense.  act: 0 none, 1 silu.
extern "C" int fe_causal_conv_act(const void* u, int dtype, long long u_stride, const float* w, const float* bias,
                                  const float* state, const int* token_seq, const int* cu_q, const int* state_slots,
                                  void* out, int tokens, int channels, int taps, int slots, int act, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS || u_stride < channels || !w || act < 0 || act > 1) return FE_BAD_ARGUMENT;
  if (taps > 1 && (!state || slots < 1)) return FE_BAD_ARGUMENT;
  if (dtype != FE_F32 && dtype != FE_BF16) return FE_BAD_ARGUMENT;
  // four channels a thread and runs of rows once that still leaves blocks for the whole chip
  const size_t element = dtype == FE_F32 ? 4 : 2;
  const bool wide = channels % 4 == 0 && u_stride % 4 == 0 && (uintptr_t)u % (4 * element) == 0 &&
                    (uintptr_t)out % (4 * element) == 0 && (long long)tokens * channels >= 4LL * SS_THREADS * 1024;
  const int vec = wide ? 4 : 1;
  const int run = wide ? 16 : 1;
  const int channel_blocks = (channels / vec + SS_THREADS - 1) / SS_THREADS;
  if (channel_blocks > 65535) return FE_BAD_ARGUMENT;
  const dim3 grid((tokens + run - 1) / run, channel_blocks);
#define LAUNCH(T, VEC)                                                                                                   \
  causal_conv_act_kernel<T, VEC><<<grid, SS_THREADS, 0, stream>>>((const T*)u, (size_t)u_stride, w, bias, state, token_seq, \
                                                                  cu_q, state_slots, (T*)out, channels, taps, slots, act, tokens, run)
  if (dtype == FE_F32) {
    if (wide) LAUNCH(float, 4); else LAUNCH(float, 1);
  } else {
    if (wide) LAUNCH(bf16_t, 4); else LAUNCH(bf16_t, 1);
  }
#undef LAUNCH
  return fe_check_launch();
}

__device__ __forceinline__ float softplus_f32(float v) { return v > 20.f ? v : log1pf(expf(v)); }

#define SS_LOG2E 1.44269504088896340736f

// The sum over the NS neighbouring lanes that share a channel (NS = 4, 8 or 16, aligned), by the data-parallel
// lane permutes: every lane of the group gets the sum.
template <int NS>
__device__ __forceinline__ float lanes_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));                  // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));                  // lane ^ 2
  if (NS >= 8) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));    // 7 - lane within 8
  if (NS >= 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // 15 - lane within 16
  return v;
}

// A segment's place in the scratch buffers: segments of one sequence start seg_len tokens apart, and a
// later sequence starts behind the last segment's first token of the one before, so the first token's
// index over seg_len plus the sequence's index counts segments without a gap's worth of collisions.
__device__ __forceinline__ int segment_id(int first_token, int seg_len, int seq) { return first_token / seg_len + seq; }

// SUMMARY false: a block walks one segment of a sequence's step from the state at the segment's start (the
// state slot for the first segment, else seg_start[id - 1]) and writes the outputs; the last segment leaves
// the state in the slot.  With seg_len beyond every step there is one segment a sequence and no scratch.
// SUMMARY true: a block walks a segment (all but a sequence's last) from a zero state without the read-out
// and leaves the state it ends with in seg_start[id] and the sum of its step sizes in seg_dt[id]:
// the recurrence is linear in the state, so the state behind the segment is
// exp(A * sum dt) * (state ahead of it) + (that end state), which scan_combine_kernel walks.
template <typename T, int NS, int R, bool SUMMARY>
__global__ __launch_bounds__(SS_THREADS) void selective_scan_kernel(
    const T* __restrict__ x, const float* __restrict__ dt_lin, const float* __restrict__ dt_bias,
    const float* __restrict__ A, const float* __restrict__ bc, size_t bc_stride, const float* __restrict__ D,
    const T* __restrict__ z, size_t z_stride, float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, T* __restrict__ out, float* __restrict__ seg_start, float* __restrict__ seg_dt,
    int C, int N, int slots, int tokens, int seg_len) {
  constexpr int CH = SS_THREADS / NS;
  __shared__ float s_dt[SS_CHUNK][CH], s_x[SS_CHUNK][CH], s_y[SS_CHUNK][CH];
  extern __shared__ float s_bc[];            // [SS_CHUNK][2 N]: a token's B row, then its C row
  const int seq = blockIdx.y;
  const int seq_begin = cu_q[seq], seq_end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (seq_end <= seq_begin || seq_end > tokens || slot < 0 || slot >= slots) return;     // an empty (padding) sequence
  const int segments = (seq_end - seq_begin + seg_len - 1) / seg_len;
  const int seg = blockIdx.z;
  if (seg >= (SUMMARY ? segments - 1 : segments)) return;
  const int begin = seq_begin + seg * seg_len, end = min(seq_end, begin + seg_len);
  const int id = segment_id(begin, seg_len, seq);
  const int tid = threadIdx.x, cl = tid / NS, part = tid % NS;
  const int c0 = blockIdx.x * CH;
  const int c = c0 + cl;
  const bool c_ok = c < C;
  const float* from = seg == 0 ? state + (size_t)slot * C * N : seg_start + (size_t)(id - 1) * C * N;
  float s[R], a[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = part * R + i;
    const bool ok = c_ok && n < N;
    s[i] = (ok && !SUMMARY) ? from[(size_t)c * N + n] : 0.f;
    a[i] = ok ? A[(size_t)c * N + n] * SS_LOG2E : 0.f;      // decays as powers of two: exp(dt A) = 2^(dt A log2 e)
  }
  const int two_n = 2 * N;
  float dt_sum = 0.f;

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
      }
    }
    for (int e = tid; e < len * two_n; e += SS_THREADS) {
      const int tt = e / two_n, j = e - tt * two_n;
      s_bc[e] = bc[(size_t)(t0 + tt) * bc_stride + j];
    }
    __syncthreads();
    // One token: the state moves on (the only step that waits for the token before: one multiply-add a
    // state), and the read-out's partial sum of this lane's states meets the other lanes' of the channel.
    // A whole chunk is unrolled, so that the decays' exponentials, the loads from LDS and the lanes'
    // exchanges of different tokens run beside one another.  The skip's term and the gate wait for the
    // chunk's end, where every thread of the block takes some of them.
    auto token = [&](int tt) {
      const float dtv = s_dt[tt][cl];
      const float dx = dtv * s_x[tt][cl];
      const float* brow = s_bc + tt * two_n;
      const float* crow = brow + N;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int n = part * R + i;
        if (n < N) {
          s[i] = fmaf(__builtin_amdgcn_exp2f(dtv * a[i]), s[i], dx * brow[n]);
          if (!SUMMARY) acc = fmaf(s[i], crow[n], acc);
        }
      }
      if (SUMMARY) {
        dt_sum += dtv;
      } else {
        acc = lanes_sum<NS>(acc);
        if (part == 0) s_y[tt][cl] = acc;
      }
    };
    if (len == SS_CHUNK) {
#pragma unroll
      for (int tt = 0; tt < SS_CHUNK; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < len; ++tt) token(tt);
    }
    if (!SUMMARY) {
      __syncthreads();
      for (int e = tid; e < len * CH; e += SS_THREADS) {
        const int tt = e / CH, cc = e - tt * CH;
        const int gc = c0 + cc;
        if (gc < C) {
          const float zv = load_as_float(z + (size_t)(t0 + tt) * z_stride + gc);
          const float y = fmaf(D[gc], s_x[tt][cc], s_y[tt][cc]);
          store_from_float(out + (size_t)(t0 + tt) * C + gc, y * (zv / (1.f + expf(-zv))));
        }
      }
    }
  }
  if (!SUMMARY && seg != segments - 1) return;
  float* to = SUMMARY ? seg_start + (size_t)id * C * N : state + (size_t)slot * C * N;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = part * R + i;
    if (c_ok && n < N) to[(size_t)c * N + n] = s[i];
  }
  if (SUMMARY && part == 0 && c_ok) seg_dt[(size_t)id * C + c] = dt_sum;
}

// From a sequence's state slot and its segments' summaries, the state at the start of every segment behind
// the first: a thread per (sequence, channel, state) walks the segments in order and overwrites each
// summary's end state with the state behind that segment.
__global__ __launch_bounds__(SS_THREADS) void scan_combine_kernel(
    const float* __restrict__ A, const float* __restrict__ state, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, float* __restrict__ seg_start, const float* __restrict__ seg_dt, int C, int N,
    int slots, int tokens, int seg_len) {
  const int seq = blockIdx.y;
  const int seq_begin = cu_q[seq], seq_end = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (seq_end <= seq_begin || seq_end > tokens || slot < 0 || slot >= slots) return;
  const int segments = (seq_end - seq_begin + seg_len - 1) / seg_len;
  const size_t e = (size_t)blockIdx.x * SS_THREADS + threadIdx.x;
  if (segments < 2 || e >= (size_t)C * N) return;
  const int c = (int)(e / N);
  const float a = A[e] * SS_LOG2E;
  float s = state[(size_t)slot * C * N + e];
  for (int seg = 0; seg + 1 < segments; ++seg) {
    const int id = segment_id(seq_begin + seg * seg_len, seg_len, seq);
    float* at = seg_start + (size_t)id * C * N + e;
    s = fmaf(__builtin_amdgcn_exp2f(a * seg_dt[(size_t)id * C + c]), s, *at);
    *at = s;
  }
}

// x [T, C] dense; dt_lin float32 [T, C] dense; dt_bias, D float32 [C]; A float32 [C, N] (negative: the decays'
// rates); bc float32 [T, >= 2 N] with row stride bc_stride (B, then C); z [T, >= C] with row stride z_stride;
// state float32 [slots, C, N]; out [T, C] dense.  lanes x per_lane >= N: lanes of a wave that share a channel
// (4, 8 or 16) and states each holds (4 with 4 or 8 lanes; 1, 2, 4, 8 or 16 with 16).
// seg_len 0: a block walks a sequence's whole step.  seg_len > 0 (a multiple of 16): a sequence's step is cut
// into segments of seg_len tokens that are walked side by side: summaries from zero states, their
// combination in order, then the outputs from every segment's true start; seg_start float32
// [segment_rows, C, N] and seg_dt float32 [segment_rows, C] are scratch with
// segment_rows >= tokens / seg_len + num_seqs + 1.
extern "C" int fe_selective_scan(const void* x, int dtype, const float* dt_lin, const float* dt_bias, const float* A,
                                 const float* bc, long long bc_stride, const float* D, const void* z, long long z_stride,
                                 float* state, const int* cu_q, const int* state_slots, void* out, int tokens, int num_seqs,
                                 int channels, int states, int slots, int lanes, int per_lane, int seg_len, float* seg_start,
                                 float* seg_dt, int segment_rows, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (channels <= 0 || states <= 0 || states > 256 || slots < 1 || bc_stride < 2LL * states || z_stride < channels ||
      lanes * per_lane < states || num_seqs > 65535)
    return FE_BAD_ARGUMENT;
  int max_segments = 1;
  if (seg_len > 0) {
    max_segments = (tokens + seg_len - 1) / seg_len;
    if (seg_len % SS_CHUNK || !seg_start || !seg_dt || segment_rows < tokens / seg_len + num_seqs + 1 || max_segments > 65535)
      return FE_BAD_ARGUMENT;
  }
  const int walk_len = seg_len > 0 ? seg_len : (1 << 30);
  const size_t lds = (size_t)SS_CHUNK * 2 * states * sizeof(float);
  const unsigned channel_blocks = (unsigned)(((long long)channels * lanes + SS_THREADS - 1) / SS_THREADS);
#define LAUNCH(T, NS, R, SUMMARY, SEGMENTS)                                                                       \
  selective_scan_kernel<T, NS, R, SUMMARY><<<dim3(channel_blocks, num_seqs, SEGMENTS), SS_THREADS, lds, stream>>>( \
      (const T*)x, dt_lin, dt_bias, A, bc, (size_t)bc_stride, D, (const T*)z, (size_t)z_stride, state, cu_q,      \
      state_slots, (T*)out, seg_start, seg_dt, channels, states, slots, tokens, walk_len)
#define SHAPES(T, SUMMARY, SEGMENTS)                                                   \
  do {                                                                                 \
    if (lanes == 4 && per_lane == 4) LAUNCH(T, 4, 4, SUMMARY, SEGMENTS);               \
    else if (lanes == 8 && per_lane == 4) LAUNCH(T, 8, 4, SUMMARY, SEGMENTS);          \
    else if (lanes == 16 && per_lane == 1) LAUNCH(T, 16, 1, SUMMARY, SEGMENTS);        \
    else if (lanes == 16 && per_lane == 2) LAUNCH(T, 16, 2, SUMMARY, SEGMENTS);        \
    else if (lanes == 16 && per_lane == 4) LAUNCH(T, 16, 4, SUMMARY, SEGMENTS);        \
    else if (lanes == 16 && per_lane == 8) LAUNCH(T, 16, 8, SUMMARY, SEGMENTS);        \
    else if (lanes == 16 && per_lane == 16) LAUNCH(T, 16, 16, SUMMARY, SEGMENTS);      \
    else return FE_BAD_ARGUMENT;                                                       \
  } while (0)
  if (dtype != FE_F32 && dtype != FE_BF16) return FE_BAD_ARGUMENT;
  if (max_segments > 1) {
    if (dtype == FE_F32) SHAPES(float, true, max_segments - 1);
    else SHAPES(bf16_t, true, max_segments - 1);
    const size_t elements = (size_t)channels * states;
    scan_combine_kernel<<<dim3((unsigned)((elements + SS_THREADS - 1) / SS_THREADS), num_seqs), SS_THREADS, 0, stream>>>(
        A, state, cu_q, state_slots, seg_start, seg_dt, channels, states, slots, tokens, walk_len);
  }
  if (dtype == FE_F32) SHAPES(float, false, max_segments);
  else SHAPES(bf16_t, false, max_segments);
#undef SHAPES
#undef LAUNCH
  return fe_check_launch();
}
