// A mixture of experts on the device: routing, the sort of (token, choice) pairs by expert, and
// two grouped matrix products over the sorted rows.  Nothing is decided on the host.
//
//   fe_moe_select:   from router logits (float32): bias added, the `top` largest per token, softmax over those alone
//                    (or, scoring 1, each chosen logit's own sigmoid)
//   fe_moe_plan:     counts per expert, their prefix sums, and the pairs ordered by expert
//   fe_moe_gate_up:  for every pair, act = min(g, L) * sigmoid(alpha min(g, L)) * (clamp(u, -L, L) + 1) with
//                    g = W_gate[e] x, u = W_up[e] x of the pair's token and expert (form 1: silu(g) * u; with
//                    input weights, g and u are first multiplied by the pair's routing weight)
//   fe_moe_down:     out[choice][token] = weight * W_down[e] act   (float32; one part per choice, so
//                    that the reader adds a token's experts up in a fixed order; the first choice's part
//                    also takes what every token gets beside its experts, a shared expert's output)
//   fe_gated_act:    the same activation over a dense [T, 2F] product (a shared expert)
//
// The grouped products tile the sorted rows within an expert (a tile never spans two experts).  float32, and
// bfloat16 with K no multiple of 32: 32 rows x 64 columns a block, K through LDS in steps of 32, FMA.  bfloat16:
// MFMA 16x16x32 over 64 rows x 64 columns with the weight straight into the operands (steps of few rows: a
// decode step streams every expert's weight once), or 64 rows x 128 columns with the weight tile through LDS like
// the rows (steps of many rows).  A launch has as many row-tile slots as the pairs could need at worst (pairs /
// rows a tile + experts); a block whose slot lies beyond the tiles there are returns at once.
#include "common.h"

// One thread per token over its row of router logits z [T, E] (float32, the product comes from the
// caller): bias added, the `top` largest chosen one after the other (the largest first; among equals
// the lowest index), weights = softmax over the chosen logits alone.
__global__ void moe_select_kernel(const float* __restrict__ z, const float* __restrict__ bias, int* __restrict__ chosen,
                                  float* __restrict__ weights, int tokens, int E, int top, int scoring) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  const float* row = z + (size_t)t * E;
  int picked[16];
  float best[16], raw[16];
  float peak = 0.f, denom = 0.f;
  for (int k = 0; k < top; ++k) {
    int arg = -1;
    float value = -INFINITY;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken = taken || picked[j] == e;
      const float v = row[e] + (bias ? bias[e] : 0.f);
      if (!taken && (arg < 0 || v > value)) {
        value = v;
        arg = e;
      }
    }
    picked[k] = arg;
    chosen[(size_t)t * top + k] = arg;
    if (k == 0) peak = value;
    raw[k] = value;
    best[k] = expf(value - peak);
    denom += best[k];
  }
  // scoring 1: a chosen expert's weight is the sigmoid of its own logit, whatever the others are
  for (int k = 0; k < top; ++k)
    weights[(size_t)t * top + k] = scoring == 1 ? 1.f / (1.f + expf(-raw[k])) : best[k] / denom;
}

extern "C" int fe_moe_select(const float* logits, const float* bias, int* chosen, float* weights, int tokens, int experts,
                             int top, int scoring, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (experts <= 0 || experts > 1024 || top < 1 || top > 16 || top > experts || scoring < 0 || scoring > 1) return FE_BAD_ARGUMENT;
  moe_select_kernel<<<(tokens + 63) / 64, 64, 0, stream>>>(logits, bias, chosen, weights, tokens, experts, top, scoring);
  return fe_check_launch();
}

// Selection by corrected scores within the best groups.  Per token: s = softmax(z) over all E experts; an
// expert's choice score is s_e + correction_e; the experts form `groups` equal runs of neighbours, a run's score is
// its largest choice score, and only experts of the `keep` best runs can be chosen (the lowest index among
// equals, for runs and for experts); the `top` largest choice scores among those are chosen, and their weights are
// their own s, divided by the sum of the chosen s (+ 1e-20), times `scale`.  The logits' rows lie `stride`
// floats apart (columns beyond E, a gate's logit say, are not read here).  One thread a token.
#define SELECT_MAX_GROUPS 64
__global__ void moe_select_grouped_kernel(const float* __restrict__ z, size_t stride, const float* __restrict__ correction,
                                          int* __restrict__ chosen, float* __restrict__ weights, int tokens, int E, int top,
                                          int groups, int keep, float scale) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  const float* row = z + (size_t)t * stride;
  float peak = -INFINITY;
  for (int e = 0; e < E; ++e) peak = fmaxf(peak, row[e]);
  float denom = 0.f;
  for (int e = 0; e < E; ++e) denom += expf(row[e] - peak);
  const float inv = 1.f / denom;
  auto score = [&](int e) { return expf(row[e] - peak) * inv; };
  auto choice = [&](int e) { return score(e) + (correction ? correction[e] : 0.f); };
  const int each = E / groups;
  unsigned long long open = ~0ull;          // bit g: run g may be chosen from
  if (keep < groups) {
    float best[SELECT_MAX_GROUPS];
    for (int g = 0; g < groups; ++g) {
      float b = -INFINITY;
      for (int e = g * each; e < (g + 1) * each; ++e) b = fmaxf(b, choice(e));
      best[g] = b;
    }
    open = 0ull;
    for (int k = 0; k < keep; ++k) {
      int arg = -1;
      float value = -INFINITY;
      for (int g = 0; g < groups; ++g)
        if (!((open >> g) & 1ull) && (arg < 0 || best[g] > value)) {
          value = best[g];
          arg = g;
        }
      open |= 1ull << arg;
    }
  }
  int picked[16];
  float own[16];
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int arg = -1;
    float value = -INFINITY;
    for (int e = 0; e < E; ++e) {
      if (!((open >> (e / each)) & 1ull)) continue;
      bool taken = false;
      for (int j = 0; j < k; ++j) taken = taken || picked[j] == e;
      if (taken) continue;
      const float v = choice(e);
      if (arg < 0 || v > value) {
        value = v;
        arg = e;
      }
    }
    picked[k] = arg;
    own[k] = score(arg);
    total += own[k];
    chosen[(size_t)t * top + k] = arg;
  }
  const float norm = scale / (total + 1e-20f);
  for (int k = 0; k < top; ++k) weights[(size_t)t * top + k] = own[k] * norm;
}

extern "C" int fe_moe_select_grouped(const float* logits, long long stride, const float* correction, int* chosen,
                                     float* weights, int tokens, int experts, int top, int groups, int keep, float scale,
                                     hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (experts <= 0 || experts > 1024 || top < 1 || top > 16 || stride < experts || groups < 1 ||
      groups > SELECT_MAX_GROUPS || experts % groups || keep < 1 || keep > groups || top > (experts / groups) * keep)
    return FE_BAD_ARGUMENT;
  moe_select_grouped_kernel<<<(tokens + 63) / 64, 64, 0, stream>>>(logits, (size_t)stride, correction, chosen, weights, tokens,
                                                                   experts, top, groups, keep, scale);
  return fe_check_launch();
}

// One block: offsets[e] = pairs of experts below e, order[offsets[e] ..] = the pairs of expert e.
// Within an expert the pairs come in no fixed order; a pair's results do not depend on its row.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ chosen, int pairs, int E,
                                                        int* __restrict__ offsets, int* __restrict__ order) {
  extern __shared__ int counts[];   // [E] counts, then [E] cursors
  int* cursor = counts + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = cursor[e] = sum;
      sum += counts[e];
    }
    offsets[E] = sum;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = chosen[i];
    if (e >= 0 && e < E) order[atomicAdd(&cursor[e], 1)] = i;
  }
}

extern "C" int fe_moe_plan(const int* chosen, int pairs, int experts, int* offsets, int* order, hipStream_t stream) {
  if (pairs <= 0) return FE_OK;
  if (experts <= 0 || experts > 1024) return FE_BAD_ARGUMENT;
  moe_plan_kernel<<<1, 1024, 2 * (size_t)experts * sizeof(int), stream>>>(chosen, pairs, experts, offsets, order);
  return fe_check_launch();
}

#define BM 32
#define BN 64
#define BK 32

// form 0: the bounded activation above; form 1: silu(g) * u.  `w` scales both products first (a router's weight
// on the expert's input: W (w x) = w (W x)).
__device__ __forceinline__ float gated(float g, float u, float limit, float alpha, int form, float w) {
  g *= w;
  u *= w;
  if (form == 1) return g / (1.f + expf(-g)) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}

// A token's first choice also takes what every token gets beside its experts (a shared expert's output,
// float32 [parts][tokens][N], added up in order first).
__device__ __forceinline__ float with_extra(float v, int choice, const float* __restrict__ extra, int parts,
                                            size_t part_stride, size_t at) {
  if (choice != 0 || !extra) return v;
  float sum = extra[at];
  for (int p = 1; p < parts; ++p) sum += extra[p * part_stride + at];
  return v + sum;
}

// The expert and the first sorted row of this block's row tile; false if the slot is beyond the tiles.
template <int ROWS = BM>
__device__ __forceinline__ bool find_tile(const int* __restrict__ offsets, int E, int slot, int& expert, int& row0,
                                          int& row_end) {
  int tiles = 0;
  for (int e = 0; e < E; ++e) {
    const int begin = offsets[e], end = offsets[e + 1];
    const int mine = (end - begin + ROWS - 1) / ROWS;
    if (slot < tiles + mine) {
      expert = e;
      row0 = begin + (slot - tiles) * ROWS;
      row_end = end;
      return true;
    }
    tiles += mine;
  }
  return false;
}

// MODE 0: rows are tokens' x gathered through the sorted pairs, the weight is [E][2N][K] (gate rows, then
// up rows), the ending is the gated activation into act [pairs, N].  MODE 1: rows are act's sorted rows,
// the weight is [E][N][K], and the result times the pair's routing weight goes to out[choice][token][N].
template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const T* __restrict__ a, const T* __restrict__ w, const int* __restrict__ offsets, const int* __restrict__ order,
    const float* __restrict__ pair_weight, T* __restrict__ act, float* __restrict__ out, int E, int N, int K, int top,
    int tokens, float limit, float alpha, int form, const float* __restrict__ extra, int extra_parts) {
  __shared__ float As[BM][BK + 1];
  __shared__ float Ws[BN][BK + 1];
  __shared__ float Us[MODE == 0 ? BN : 1][BK + 1];
  __shared__ int pair_of[BM];
  int expert, row0, row_end;
  if (!find_tile(offsets, E, blockIdx.x, expert, row0, row_end)) return;
  const int tid = threadIdx.x;
  const int n0 = blockIdx.y * BN;
  if (tid < BM) pair_of[tid] = row0 + tid < row_end ? order[row0 + tid] : -1;
  __syncthreads();
  const int ty = tid / 16, tx = tid % 16;
  float acc_g[2][4], acc_u[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc_g[i][j] = acc_u[i][j] = 0.f;
  const size_t w_rows = MODE == 0 ? 2 * (size_t)N : (size_t)N;
  const T* w_expert = w + (size_t)expert * w_rows * K;

  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int e = tid; e < BM * BK; e += 256) {
      const int r = e / BK, k = e % BK;
      float v = 0.f;
      const int pair = pair_of[r];
      if (pair >= 0 && k0 + k < K) {
        const size_t src = MODE == 0 ? (size_t)(pair / top) : (size_t)(row0 + r);
        v = load_as_float(a + src * K + k0 + k);
      }
      As[r][k] = v;
    }
    for (int e = tid; e < BN * BK; e += 256) {
      const int n = e / BK, k = e % BK;
      const bool ok = n0 + n < N && k0 + k < K;
      Ws[n][k] = ok ? load_as_float(w_expert + (size_t)(n0 + n) * K + k0 + k) : 0.f;
      if (MODE == 0) Us[n][k] = ok ? load_as_float(w_expert + ((size_t)N + n0 + n) * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < BK; ++k) {
      const float a0 = As[ty * 2][k], a1 = As[ty * 2 + 1][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float wv = Ws[tx + 16 * j][k];
        acc_g[0][j] = fmaf(a0, wv, acc_g[0][j]);
        acc_g[1][j] = fmaf(a1, wv, acc_g[1][j]);
        if (MODE == 0) {
          const float uv = Us[tx + 16 * j][k];
          acc_u[0][j] = fmaf(a0, uv, acc_u[0][j]);
          acc_u[1][j] = fmaf(a1, uv, acc_u[1][j]);
        }
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = ty * 2 + i;
    const int pair = pair_of[r];
    if (pair < 0) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      if (MODE == 0) {
        store_from_float(act + (size_t)(row0 + r) * N + n, gated(acc_g[i][j], acc_u[i][j], limit, alpha, form, pair_weight ? pair_weight[pair] : 1.f));
      } else {
        const int token = pair / top, choice = pair - token * top;
        out[((size_t)choice * tokens + token) * N + n] =
            with_extra(acc_g[i][j] * (pair_weight ? pair_weight[pair] : 1.f), choice, extra, extra_parts, (size_t)tokens * N, (size_t)token * N + n);
      }
    }
  }
}

// The same two products on the matrix cores, for bfloat16 with K a multiple of 32: a block takes 64 sorted
// rows of one expert and 64 output columns (MODE 0: 64 gate columns and their 64 up columns), K in steps
// of 32.  The rows go through LDS (two stages, one barrier a step; rows 80 bytes apart so that the
// 16-byte reads of a fragment spread over the banks), the weight goes straight from memory into the
// MFMA operand: wave w owns columns 16 w .. 16 w + 15 and all four 16-row tiles.  Both operands of the
// next step are requested before this step's products.  A result lane holds rows 4 (lane / 16) + i of a
// tile at column lane % 16.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;
#define TM 64
#define TN 64
#define TK 32
#define TPAD 40

// A barrier that orders the block's LDS traffic only: the loads from global memory that are under way for
// later steps stay under way (a barrier that fences every address space waits for all of them, and the
// operands requested steps ahead would arrive no earlier than those of the step at hand).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int MODE, int NT, int MT>
__global__ __launch_bounds__(256) void moe_grouped_mfma_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ offsets,
    const int* __restrict__ order, const float* __restrict__ pair_weight, bf16_t* __restrict__ act,
    float* __restrict__ out, int E, int N, int K, int top, int tokens, float limit, float alpha, int form,
    const float* __restrict__ extra, int extra_parts, int slots, int column_tiles) {
  // NT: groups of 16 columns a wave (a block takes 64 NT columns); MT: tiles of 16 rows a wave (a block takes
  // 16 MT rows, every wave all of them).  Steps of few rows launch <MODE, 1, 4>: many blocks, each streaming
  // its part of the weight.  For steps of many rows the larger shapes of this kernel were measured and lost to
  // the kernel below, whose weight tile goes through LDS (<MODE, 2, 4>: 3.80 against 3.67 ms for a prompt of 2,048
  // tokens at a width of 2,048; <MODE, 2, 8> at 4,096: 9.9 against 9.6 ms; eight waves over 128 rows, the second
  // four asking for the weight fragments of the first four: 4.3 ms at 2,048).
  constexpr int ROWS = 16 * MT;
  constexpr int AL = ROWS / 64;          // 16-byte pieces of a step's rows a thread brings
  __shared__ __attribute__((aligned(16))) bf16_t As[2][ROWS][TPAD];
  __shared__ int pair_of[ROWS];
  // Blocks go to the eight dies (XCDs, each with an L2 of its own) in turn by their index.  The row tiles of
  // one expert under one column tile read the same part of the weight, so they are made neighbours in the
  // order of work (the row slot runs fastest) and a die takes a run of that order: block b works on item
  // (b % 8) * ceil(items / 8) + b / 8, and a weight tile comes from memory once for all its row tiles.
  const int items = slots * column_tiles;
  const int per_die = (items + 7) / 8;
  const int item = (int)(blockIdx.x % 8) * per_die + (int)(blockIdx.x / 8);
  if (item >= items) return;
  int expert, row0, row_end;
  if (!find_tile<ROWS>(offsets, E, item % slots, expert, row0, row_end)) return;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 16, lq = lane / 16;
  const int n0 = (item / slots) * (TN * NT);
  for (int r = tid; r < ROWS; r += 256) pair_of[r] = row0 + r < row_end ? order[row0 + r] : -1;
  __syncthreads();
  // this thread's 16-byte pieces of a step's rows: rows tid / 4 + 64 j, k chunk tid % 4
  const int my_chunk = tid % 4;
  int my_row[AL];
  bool my_live[AL];
  const bf16_t* a_at[AL];
#pragma unroll
  for (int j = 0; j < AL; ++j) {
    my_row[j] = tid / 4 + 64 * j;
    const int pair = pair_of[my_row[j]];
    my_live[j] = pair >= 0;
    const size_t src = pair < 0 ? 0 : (MODE == 0 ? (size_t)(pair / top) : (size_t)(row0 + my_row[j]));
    a_at[j] = a + src * K + my_chunk * 8;
  }
  const size_t w_rows = MODE == 0 ? 2 * (size_t)N : (size_t)N;
  int n[NT];
  const bf16_t* wg_at[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    n[nt] = n0 + (wave * NT + nt) * 16 + lr;
    wg_at[nt] = w + ((size_t)expert * w_rows + min(n[nt], N - 1)) * K + lq * 8;
  }
  const size_t up_offset = MODE == 0 ? (size_t)N * K : 0;
  floatx4 acc_g[NT][MT], acc_u[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc_g[nt][mt] = acc_u[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const uintx4 zero = {0u, 0u, 0u, 0u};
  // Step s has its operands in register set s % DEPTH, requested DEPTH steps ahead (a step's arithmetic is far
  // shorter than a trip to memory, and a launch of few blocks keeps the memory busy only through what each
  // block has in flight).  The rows of step s + 1 go into the other LDS stage while step s multiplies; one
  // barrier a step.  Whole rounds of DEPTH steps are straight-line code; steps beyond the last fetch the last
  // step's operands again, so that no load stands under a branch.
  constexpr int DEPTH = MT > 4 ? 2 : 4;
  const int steps = K / TK;
  uintx4 a_reg[DEPTH][AL], wg_reg[DEPTH][NT], wu_reg[DEPTH][NT];
  auto fetch = [&](int step, int set) {
    const int at = min(step, steps - 1) * TK;
#pragma unroll
    for (int j = 0; j < AL; ++j) a_reg[set][j] = *(const uintx4*)(a_at[j] + at);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      wg_reg[set][nt] = *(const uintx4*)(wg_at[nt] + at);
      if (MODE == 0) wu_reg[set][nt] = *(const uintx4*)(wg_at[nt] + up_offset + at);
    }
  };
  auto multiply = [&](int stage, int set) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 rows = *(const bf16x8*)&As[stage][mt * 16 + lr][lq * 8];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc_g[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, __builtin_bit_cast(bf16x8, wg_reg[set][nt]), acc_g[nt][mt], 0, 0, 0);
        if (MODE == 0)
          acc_u[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, __builtin_bit_cast(bf16x8, wu_reg[set][nt]), acc_u[nt][mt], 0, 0, 0);
      }
    }
  };
  auto stash = [&](int stage, int set) {
#pragma unroll
    for (int j = 0; j < AL; ++j) *(uintx4*)&As[stage][my_row[j]][my_chunk * 8] = my_live[j] ? a_reg[set][j] : zero;
  };
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) fetch(u, u);
  stash(0, 0);
  lds_barrier();
  int step = 0;
  for (; step + DEPTH <= steps; step += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      multiply(u & 1, u);
      stash((u + 1) & 1, (u + 1) % DEPTH);
      fetch(step + u + DEPTH, u);
      lds_barrier();
    }
  }
  const int left = steps - step;       // 0 .. DEPTH - 1, the same for every thread
#pragma unroll
  for (int u = 0; u < DEPTH - 1; ++u)
    if (u < left) {
      multiply(u & 1, u);
      stash((u + 1) & 1, (u + 1) % DEPTH);
      lds_barrier();
    }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (n[nt] >= N) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = mt * 16 + lq * 4 + i;
        const int pair = pair_of[r];
        if (pair < 0) continue;
        if (MODE == 0) {
          act[(size_t)(row0 + r) * N + n[nt]] = float_to_bf16(gated(acc_g[nt][mt][i], acc_u[nt][mt][i], limit, alpha, form, pair_weight ? pair_weight[pair] : 1.f));
        } else {
          const int token = pair / top, choice = pair - token * top;
          out[((size_t)choice * tokens + token) * N + n[nt]] = with_extra(
              acc_g[nt][mt][i] * (pair_weight ? pair_weight[pair] : 1.f), choice, extra, extra_parts, (size_t)tokens * N, (size_t)token * N + n[nt]);
        }
      }
  }
}

// The shape for steps of many rows: the weight tile goes through LDS as the rows do.  Straight into the MFMA
// operand, a lane asks for 16 bytes of a weight row of its own, and the 64 lanes of a load are 64 accesses of
// the CU's L1 (measured: 80 million a launch, 312,000 a CU in 473,000 cycles, with the matrix cores busy 14 %);
// here four neighbouring lanes bring 64 neighbouring bytes of one weight row, a quarter of the accesses, and every
// wave reads its fragments out of LDS.  Block = 64 rows x 128 columns (MODE 0: and their 128 up columns), K in
// steps of 32, two stages, operands requested DEPTH steps ahead, one LDS-only barrier a step.  (Rows of 64 bytes
// with their 16-byte pieces exchanged by the row's number, instead of rows 80 bytes apart, took the bank conflicts
// from 20 million cycles a launch to none and the launch from 179 to 181 us: they were not what it waits for.
// Rows and weight tile straight from global memory into LDS (`global_load_lds_dwordx4`, no staging registers,
// three and four steps deep) gave 3.85 instead of 3.64 ms for a prompt of 2,048 tokens at a width of 2,048.  With
// the products taken out of this kernel its loads, LDS stores and barriers alone take 124 of the 174 us, and with
// every block reading the same hot tile 151: neither the depth of the prefetch nor where the bytes come from
// is what bounds it.  Blocks of 128 rows in this shape need the registers of a whole SIMD a wave: 4.25 ms.)
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_staged_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ offsets,
    const int* __restrict__ order, const float* __restrict__ pair_weight, bf16_t* __restrict__ act,
    float* __restrict__ out, int E, int N, int K, int top, int tokens, float limit, float alpha, int form,
    const float* __restrict__ extra, int extra_parts, int slots, int column_tiles) {
  constexpr int COLS = 128, MATS = MODE == 0 ? 2 : 1, NT = 2, MT = 4;
  __shared__ __attribute__((aligned(16))) bf16_t As[2][TM][TPAD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][MATS][COLS][TPAD];
  __shared__ int pair_of[TM];
  const int items = slots * column_tiles;
  const int per_die = (items + 7) / 8;
  const int item = (int)(blockIdx.x % 8) * per_die + (int)(blockIdx.x / 8);
  if (item >= items) return;
  int expert, row0, row_end;
  if (!find_tile<TM>(offsets, E, item % slots, expert, row0, row_end)) return;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, lr = lane % 16, lq = lane / 16;
  const int n0 = (item / slots) * COLS;
  if (tid < TM) pair_of[tid] = row0 + tid < row_end ? order[row0 + tid] : -1;
  __syncthreads();
  // a thread's 16-byte pieces of a step: row tid / 4 of the rows, weight rows tid / 4 and tid / 4 + 64 of each
  // matrix, k chunk tid % 4
  const int my_row = tid / 4, my_chunk = tid % 4;
  const int my_pair = pair_of[my_row];
  const size_t src = my_pair < 0 ? 0 : (MODE == 0 ? (size_t)(my_pair / top) : (size_t)(row0 + my_row));
  const bf16_t* a_at = a + src * K + my_chunk * 8;
  const size_t w_rows = MODE == 0 ? 2 * (size_t)N : (size_t)N;
  const bf16_t* w_at[MATS][2];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      w_at[m][j] = w + ((size_t)expert * w_rows + (size_t)m * N + min(n0 + my_row + 64 * j, N - 1)) * K + my_chunk * 8;
  floatx4 acc[MATS][NT][MT];
#pragma unroll
  for (int m = 0; m < MATS; ++m)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[m][nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const uintx4 zero = {0u, 0u, 0u, 0u};
  constexpr int DEPTH = MODE == 0 ? 2 : 4;      // with two matrices the registers hold two steps' operands beside the sums
  const int steps = K / TK;
  uintx4 a_reg[DEPTH], w_reg[DEPTH][MATS][2];
  auto fetch = [&](int step, int set) {
    const int at = min(step, steps - 1) * TK;
    a_reg[set] = *(const uintx4*)(a_at + at);
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int j = 0; j < 2; ++j) w_reg[set][m][j] = *(const uintx4*)(w_at[m][j] + at);
  };
  auto stash = [&](int stage, int set) {
    *(uintx4*)&As[stage][my_row][my_chunk * 8] = my_pair < 0 ? zero : a_reg[set];
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int j = 0; j < 2; ++j) *(uintx4*)&Ws[stage][m][my_row + 64 * j][my_chunk * 8] = w_reg[set][m][j];
  };
  auto multiply = [&](int stage) {
    bf16x8 cols[MATS][NT];
#pragma unroll
    for (int m = 0; m < MATS; ++m)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) cols[m][nt] = *(const bf16x8*)&Ws[stage][m][(wave * NT + nt) * 16 + lr][lq * 8];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 rows = *(const bf16x8*)&As[stage][mt * 16 + lr][lq * 8];
#pragma unroll
      for (int m = 0; m < MATS; ++m)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[m][nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rows, cols[m][nt], acc[m][nt][mt], 0, 0, 0);
    }
  };
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) fetch(u, u);
  stash(0, 0);
  lds_barrier();
  int step = 0;
  for (; step + DEPTH <= steps; step += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      // set u went into LDS during the step before: its registers are free, and what is asked for now has
      // this step's products and the next step's to arrive in
      fetch(step + u + DEPTH, u);
      multiply(u & 1);
      stash((u + 1) & 1, (u + 1) % DEPTH);
      lds_barrier();
    }
  }
  const int left = steps - step;
#pragma unroll
  for (int u = 0; u < DEPTH - 1; ++u)
    if (u < left) {
      multiply(u & 1);
      stash((u + 1) & 1, (u + 1) % DEPTH);
      lds_barrier();
    }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + (wave * NT + nt) * 16 + lr;
    if (n >= N) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = mt * 16 + lq * 4 + i;
        const int pair = pair_of[r];
        if (pair < 0) continue;
        if (MODE == 0) {
          act[(size_t)(row0 + r) * N + n] = float_to_bf16(gated(acc[0][nt][mt][i], acc[MATS - 1][nt][mt][i], limit, alpha, form, pair_weight ? pair_weight[pair] : 1.f));
        } else {
          const int token = pair / top, choice = pair - token * top;
          out[((size_t)choice * tokens + token) * N + n] = with_extra(
              acc[0][nt][mt][i] * (pair_weight ? pair_weight[pair] : 1.f), choice, extra, extra_parts, (size_t)tokens * N, (size_t)token * N + n);
        }
      }
  }
}

// Two groups of columns a wave from this many pairs on (the launch then still has blocks enough).
#define WIDE_COLUMNS_MIN_PAIRS 1024

// blocks of a launch: the items rounded up to a whole number a die
static unsigned mfma_blocks(int slots, int column_tiles) { return (unsigned)(((long long)slots * column_tiles + 7) / 8 * 8); }

// Which shape a launch takes: from WIDE_COLUMNS_MIN_PAIRS pairs on the one whose weight tile goes through LDS
// (a prompt of 2,048 tokens at a width of 2,048: 3.80 -> 3.67 ms against the direct shape with two column groups
// a wave; at 4,096: 10.0 -> 9.6 ms, where the direct shape with blocks of 128 rows reached 9.9), below that the
// direct shape with one column group a wave, which streams the weight at 3 to 4.7 TB/s in a decode step.
#define MFMA_LAUNCH(MODE, COLUMNS, A, W, PW, ACT, OUT, N_, K_, LIMIT, ALPHA, FORM, EXTRA, EXTRA_PARTS)                        \
  do {                                                                                                                   \
    const bool wide = pairs >= WIDE_COLUMNS_MIN_PAIRS;                                                                   \
    const int slots = (int)(pairs / TM + experts);                                                                       \
    const int tiles = ((COLUMNS) + (wide ? 2 : 1) * TN - 1) / ((wide ? 2 : 1) * TN);                                      \
    if (wide)                                                                                                            \
      moe_grouped_staged_kernel<MODE><<<mfma_blocks(slots, tiles), 256, 0, stream>>>(                                    \
          A, W, offsets, order, PW, ACT, OUT, experts, N_, K_, top, tokens, LIMIT, ALPHA, FORM, EXTRA, EXTRA_PARTS, slots, tiles); \
    else                                                                                                                 \
      moe_grouped_mfma_kernel<MODE, 1, 4><<<mfma_blocks(slots, tiles), 256, 0, stream>>>(                                \
          A, W, offsets, order, PW, ACT, OUT, experts, N_, K_, top, tokens, LIMIT, ALPHA, FORM, EXTRA, EXTRA_PARTS, slots, tiles); \
  } while (0)

static bool mfma_fits(const void* a, const void* w, int K) {
  return K % TK == 0 && ((((uintptr_t)a) | ((uintptr_t)w)) & 15) == 0;
}

extern "C" int fe_moe_gate_up(const void* x, const void* gate_up, int dtype, const int* offsets, const int* order, void* act,
                              int tokens, int top, int experts, int hidden, int inner, float limit, float alpha, int form,
                              const float* input_weight, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (top < 1 || experts < 1 || experts > 1024 || hidden <= 0 || inner <= 0 || form < 0 || form > 1 ||
      (form == 0 && !(limit > 0.f)))
    return FE_BAD_ARGUMENT;
  const long long pairs = (long long)tokens * top;
  const dim3 grid((unsigned)(pairs / BM + experts), (unsigned)((inner + BN - 1) / BN));
  if (dtype == FE_F32)
    moe_grouped_kernel<float, 0><<<grid, 256, 0, stream>>>((const float*)x, (const float*)gate_up, offsets, order, input_weight,
                                                           (float*)act, nullptr, experts, inner, hidden, top, tokens, limit, alpha, form, nullptr, 0);
  else if (dtype == FE_BF16 && mfma_fits(x, gate_up, hidden)) {
    MFMA_LAUNCH(0, inner, (const bf16_t*)x, (const bf16_t*)gate_up, input_weight, (bf16_t*)act, nullptr, inner, hidden, limit, alpha, form, nullptr, 0);
  } else if (dtype == FE_BF16)
    moe_grouped_kernel<bf16_t, 0><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)gate_up, offsets, order, input_weight,
                                                            (bf16_t*)act, nullptr, experts, inner, hidden, top, tokens, limit,
                                                            alpha, form, nullptr, 0);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

extern "C" int fe_moe_down(const void* act, const void* down, int dtype, const int* offsets, const int* order,
                           const float* pair_weight, float* out, int tokens, int top, int experts, int hidden, int inner,
                           const float* extra, int extra_parts, hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (top < 1 || experts < 1 || experts > 1024 || hidden <= 0 || inner <= 0 || (extra && extra_parts < 1)) return FE_BAD_ARGUMENT;
  const long long pairs = (long long)tokens * top;
  const dim3 grid((unsigned)(pairs / BM + experts), (unsigned)((hidden + BN - 1) / BN));
  if (dtype == FE_F32)
    moe_grouped_kernel<float, 1><<<grid, 256, 0, stream>>>((const float*)act, (const float*)down, offsets, order, pair_weight,
                                                           nullptr, out, experts, hidden, inner, top, tokens, 0.f, 0.f, 0, extra,
                                                           extra_parts);
  else if (dtype == FE_BF16 && mfma_fits(act, down, inner)) {
    MFMA_LAUNCH(1, hidden, (const bf16_t*)act, (const bf16_t*)down, pair_weight, nullptr, out, hidden, inner, 0.f, 0.f, 0, extra, extra_parts);
  } else if (dtype == FE_BF16)
    moe_grouped_kernel<bf16_t, 1><<<grid, 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)down, offsets, order, pair_weight,
                                                            nullptr, out, experts, hidden, inner, top, tokens, 0.f, 0.f, 0, extra,
                                                           extra_parts);
  else
    return FE_BAD_ARGUMENT;
  return fe_check_launch();
}

// ---------------------------------------------------------------- the activation over a dense product
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gate_up, T* __restrict__ out, long long count, int inner, float limit,
                                 float alpha) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const long long t = i / inner;
  const int n = (int)(i - t * inner);
  const T* row = gate_up + t * 2 * inner;
  store_from_float(out + i, gated(load_as_float(row + n), load_as_float(row + inner + n), limit, alpha, 0, 1.f));
}

extern "C" int fe_gated_act(const void* gate_up, void* out, int dtype, int tokens, int inner, float limit, float alpha,
                            hipStream_t stream) {
  if (tokens <= 0) return FE_OK;
  if (inner <= 0 || !(limit > 0.f)) return FE_BAD_ARGUMENT;
  const long long count = (long long)tokens * inner;
  const int blocks = (int)((count + 255) / 256);
  if (dtype == FE_F32) gated_act_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, count, inner, limit, alpha);
  else if (dtype == FE_BF16) gated_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, count, inner, limit, alpha);
  else return FE_BAD_ARGUMENT;
  return fe_check_launch();
}
