// Causal attention of many query heads over one shared cache of rows, on the matrix cores (bfloat16).
//
// Every head of a token reads the same cached rows: a row of DK numbers is the key of all heads, and
// its first DV numbers, kept a second time in transposed pages, are the value (attention through a
// latent, after the queries were taken through the keys' up-projection).  Key pages
// [page][1][slot][DK], value pages [page][1][DV][slot]; the step's own rows are already in them.
//
// Block = 4 waves on 64 query rows of one sequence, a row being a (token, head) pair, token-major, so
// that the 64 rows of a block share their keys; a wave owns 16 rows.  Keys are walked in tiles of 32:
// the tile's keys and its transposed values reach LDS by `global_load_lds_dwordx4` (64 lanes x 16 bytes at
// consecutive LDS addresses, no staging registers: every load of a tile is in flight at once), and all
// four waves read their MFMA operands from there.  Which global bytes a lane loads is free, where they
// land is not, so a key row's 16-byte chunks lie permuted by the row's low bits and a value dim's four
// key chunks by the dim's bits 2 and 3: the operand reads of 16 lanes then spread over the banks.  Two
// buffers: a tile's loads run under the products of the tile before.  S^T = K Q^T and O^T = V^T P^T on MFMA 16x16x32 with
// scores, statistics and outputs in registers: lane (r = lane % 16, g = lane / 16) holds, of row r,
// the scores of keys 8g .. 8g + 7 of the tile (the key rows of the first product are permuted so that
// they come out that way, which is the order the second product's operands want) and the outputs of
// dims 16t + 4g .. + 3 of every tile t of 16 dims.  Online softmax in base 2, float32.
//
// A launch may cut every block's keys into `splits` runs of whole tiles (grid.y) for steps with few
// rows and long contexts; each run leaves its unnormalised output, maximum and sum in float32, and a
// second kernel merges them in order.  Slots beyond the context may hold anything: their values are
// masked to zero in the operand.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) unsigned int uintx4;
typedef __attribute__((ext_vector_type(2))) unsigned int uintx2;

#define LA_KEYS 32
#define LA_ROWS 64

__device__ __forceinline__ unsigned int pack_two(float lo, float hi) {
  return (unsigned int)float_to_bf16(lo) | ((unsigned int)float_to_bf16(hi) << 16);
}

// Where chunk `slot` of key row `key` lies in the row's LDS image (and the other way round: the map is its
// own inverse).  The 16 rows that one operand read touches are rows 8a + b (+ 4h), a and b below 4; rows are
// CHUNKS units of 16 bytes apart, which moves odd rows by 8 units mod 16 where CHUNKS is 8 mod 16, and
// 4a + b with its bit 3 flipped for odd b, XORed into the chunk index, puts the 16 rows on 16 distinct
// units mod 16, that is on all banks once.  A row's last chunks, where they do not fill a group of 16, are
// permuted within their own group of 8 (or 4) only.
template <int CHUNKS>
__device__ __forceinline__ int key_chunk(int key, int slot) {
  constexpr int WHOLE = CHUNKS & ~15, REST = CHUNKS & 15;
  constexpr int REST_MASK = REST % 8 == 0 ? 7 : (REST % 4 == 0 ? 3 : (REST % 2 == 0 ? 1 : 0));
  int s = ((key >> 3) & 3) * 4 + (key & 3);
  if (CHUNKS % 16 == 8) s ^= (key & 1) << 3;
  return slot ^ (slot < WHOLE ? s : (s & REST_MASK));
}

// 16 bytes from the LDS byte address `at` + OFFSET (an immediate of the instruction); nothing waits for them here
template <int OFFSET>
__device__ __forceinline__ uintx4 lds_read16(unsigned int at) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "the instruction's offset field");
  uintx4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(OFFSET) : "memory");
  return v;
}
// wait until at most `pending` of this wave's LDS reads are outstanding; `v` is what the wait is for (LDS reads
// return in order; whatever else is under way on the same counter makes such a wait stricter, never weaker)
template <int PENDING>
__device__ __forceinline__ void lds_arrived(uintx4& v) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
}
#define LA_AHEAD 4      // operand reads in flight ahead of the product that uses them
#define LA_RING 8

// body(integral constant I) for I = FROM .. TO - 1: a loop whose counter is a constant expression in its body
template <int I> struct index_constant { static constexpr int value = I; };
template <int FROM, int TO, typename Body>
__device__ __forceinline__ void static_for(Body&& body) {
  if constexpr (FROM < TO) {
    body(index_constant<FROM>{});
    static_for<FROM + 1, TO>(body);
  }
}

// Fragment F of the first product's key operand (step F / 2 of the dims, half F % 2 of the tile's keys) from the
// key image at LDS byte address `keys_at`.  The lane's chunk of step c is 4c + lq, at slot (4c + lq) ^ s of its
// row, s below 16 and lq below 4: the slot is (4c & ~15) + ((4c & 15) ^ lq ^ s), so `at` holds, per half, the
// row's byte offset plus 16 ((4j) ^ lq ^ s) for j = 0 .. 3 (entries 0 .. 3), and the same with s cut to the
// row's last, smaller group of chunks (entries 4 .. 7); the rest is an immediate of the instruction.
template <int CHUNKS, int F>
__device__ __forceinline__ uintx4 key_fragment(unsigned int keys_at, const unsigned int (&at)[2][8]) {
  constexpr int c = F >> 1, h = F & 1, first = 4 * c;
  constexpr bool rest = first >= (CHUNKS & ~15);
  return lds_read16<(first & ~15) * 16>(keys_at + at[h][(rest ? 4 : 0) + ((first & 15) >> 2)]);
}

__device__ __forceinline__ void tile_to_lds(const void* global, void* lds) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)global,
                                   (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// Queries (DK / 8 registers a lane) and outputs (DV / 4) stay in registers for the whole walk: the sizes that need
// more than half a SIMD's registers for them run one block a CU, the others two.
template <int DK, int DV>
__global__ __launch_bounds__(256, (DK / 8 + DV / 4 > 160) ? 1 : 2) void latent_attention_kernel(
    const bf16_t* __restrict__ q, size_t q_stride, const bf16_t* __restrict__ key_pages,
    const bf16_t* __restrict__ value_pages, bf16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int* __restrict__ cu_q, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int table_stride, int heads, int block_shift, int num_blocks,
    float scale_log2, int splits, int total_rows) {
  constexpr int KC = DK / 32, DT = DV / 16, CHUNKS = DK / 8;
  constexpr int K_UNITS = LA_KEYS * CHUNKS, V_UNITS = DV * 4;             // 16-byte units of a tile's keys and values
  constexpr int LOADS = (K_UNITS + V_UNITS) / 64;                         // load instructions a tile, 64 units each
  constexpr int MINE = (LOADS + 3) / 4;                                   // ... of which a wave issues this many
  constexpr int TILE_BYTES = (K_UNITS + V_UNITS) * 16;                    // one buffer
  static_assert(DT >= LA_AHEAD && 2 * KC >= LA_AHEAD, "the rings of operand reads");
  static_assert(K_UNITS % 64 == 0 && V_UNITS % 64 == 0, "whole load instructions");
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_lds[];
  // a buffer: K_UNITS units of keys (unit u: key u / CHUNKS, chunk key_chunk(key, u % CHUNKS) of it), then V_UNITS units of
  // values (unit u: dim u / 4, keys 8 ((u % 4) ^ (dim >> 2 & 3)) .. + 7 of the tile)

  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 15, lq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int seq = blockIdx.z, split = blockIdx.y;
  const int q0 = cu_q[seq];
  const int q_len = cu_q[seq + 1] - q0;
  const int ctx = ctx_len[seq];
  const int before = ctx - q_len;
  const int rows_total = q_len * heads;
  const int row0 = (gridDim.x - 1 - blockIdx.x) * LA_ROWS;      // a sequence's last rows walk the most keys: they start first
  if (row0 >= rows_total || before < 0) return;

  const int my_row = row0 + wave * 16 + lr;
  const bool row_ok = my_row < rows_total;
  const int tok = row_ok ? my_row / heads : 0;
  const int head = row_ok ? my_row - tok * heads : 0;
  const int pos = before + tok;
  const bool wave_ok = row0 + wave * 16 < rows_total;
  const int wave_pos_max = before + (min(rows_total, row0 + wave * 16 + 16) - 1) / heads;
  const int block_pos_max = before + (min(rows_total, row0 + LA_ROWS) - 1) / heads;
  const int tiles = block_pos_max / LA_KEYS + 1;
  const int run = (tiles + splits - 1) / splits;
  const int t_lo = split * run, t_hi = min(tiles, t_lo + run);

  bf16x8 qb[KC];
  {
    const bf16_t* qrow = q + (size_t)(q0 + tok) * q_stride + (size_t)head * DK + lq * 8;
#pragma unroll
    for (int c = 0; c < KC; ++c)
      qb[c] = row_ok ? *(const bf16x8*)(qrow + c * 32) : __builtin_bit_cast(bf16x8, uintx4{0u, 0u, 0u, 0u});
  }
  floatx4 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  const int* table = block_table + (size_t)seq * table_stride;
  const int last_key = ctx - 1;

  // One tile's loads: the wave's share of them.  Keys beyond the context read the last key's page (their
  // scores are masked and their values cleared in the operand), so every address is a valid one.  What does
  // not change from tile to tile is worked out once: which key of the tile a lane's load n fetches and where
  // in that key's row (or value dim) it starts.  The page ids of a tile are fetched a tile ahead, behind the
  // loads of the tile before: a wait for a page id right before its load would stall every tile.
  const int block_size = 1 << block_shift, slot_mask = block_size - 1;
  int rel[MINE], off[MINE], lim[MINE], page_id[MINE];
#pragma unroll
  for (int n = 0; n < MINE; ++n) {
    const int load = min(wave + 4 * n, LOADS - 1);
    const int u = load * 64 + lane;
    if (load < K_UNITS / 64) {
      const int key = u / CHUNKS, slot = u - key * CHUNKS;
      rel[n] = key;
      off[n] = key_chunk<CHUNKS>(key, slot) * 8;
      lim[n] = last_key;
    } else {
      const int uv = u - K_UNITS;
      const int dim = uv >> 2, kc = (uv & 3) ^ ((dim >> 2) & 3);
      rel[n] = 8 * kc;
      off[n] = dim << block_shift;
      lim[n] = last_key & ~7;
    }
  }
  auto page_ids = [&](int tile) {
#pragma unroll
    for (int n = 0; n < MINE; ++n) page_id[n] = table[min(tile * LA_KEYS + rel[n], lim[n]) >> block_shift];
  };
  auto fetch = [&](int tile, int buffer) {
    const int kb = tile * LA_KEYS;
#pragma unroll
    for (int n = 0; n < MINE; ++n) {
      const int load = wave + 4 * n;
      if (load < LOADS) {
        const int kp = min(kb + rel[n], lim[n]);
        const size_t page = (size_t)min(max(page_id[n], 0), num_blocks - 1);
        const bf16_t* src = load < K_UNITS / 64 ? key_pages + ((page << block_shift) + (kp & slot_mask)) * DK + off[n]
                                                : value_pages + ((page * DV) << block_shift) + off[n] + (kp & slot_mask);
        tile_to_lds(src, tile_lds + buffer * TILE_BYTES + load * 1024);
      }
    }
  };
  const unsigned int lds_at = (unsigned int)(size_t)(const __attribute__((address_space(3))) unsigned char*)tile_lds;
  // where this lane's operand reads start within a buffer (see key_fragment); operand row lr of half h is key
  // 8 (lr / 4) + 4 h + lr % 4, so that result row 4 g + i is key 8 g + 4 h + i
  unsigned int key_at[2][8];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int key = 8 * (lr >> 2) + 4 * h + (lr & 3);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      key_at[h][j] = (unsigned int)((key * CHUNKS + (key_chunk<CHUNKS>(key, 4 * j + lq) & 15)) * 16);
      const int r = 4 * j + lq < (CHUNKS & 15) ? 4 * j + lq : 0;        // entries beyond the row's last group are never read
      key_at[h][4 + j] = (unsigned int)((key * CHUNKS + (key_chunk<CHUNKS>(key, (CHUNKS & ~15) + r) & 15)) * 16);
    }
  }
  const unsigned int value_at = (unsigned int)((lr * 4 + (lq ^ ((lr >> 2) & 3))) * 16);

  // Two buffers: a tile's loads are issued before the tile before it is multiplied, and land meanwhile.  The
  // operands are read from LDS by inline assembly with their waits written out: the compiler, with loads
  // into LDS in flight, would wait for all of them before its first LDS read.
  if (t_lo < t_hi) {
    page_ids(t_lo);
    fetch(t_lo, 0);
    page_ids(t_lo + 1);
  }
  for (int tile = t_lo; tile < t_hi; ++tile) {
    const int kb = tile * LA_KEYS;
    const int buffer = (tile - t_lo) & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wave's loads of the tile have landed
    __syncthreads();                                        // ... and everyone's; the other buffer's tile is consumed
    if (tile + 1 < t_hi) {
      fetch(tile + 1, buffer ^ 1);
      page_ids(tile + 2);         // keys beyond the context read the last key's entry: always a valid index
    }
    if (!wave_ok || kb > wave_pos_max) continue;            // the whole wave: no row, or no row that sees this tile
    const unsigned int keys_at = lds_at + buffer * TILE_BYTES, values_at = keys_at + K_UNITS * 16;

    floatx4 st[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    {
      constexpr int FRAGMENTS = 2 * KC;       // step c outermost, half h inside
      uintx4 ring[LA_RING];
      static_for<0, LA_AHEAD>([&](auto f) { ring[f.value] = key_fragment<CHUNKS, f.value>(keys_at, key_at); });
      static_for<0, FRAGMENTS>([&](auto fc) {
        constexpr int f = fc.value;
        if constexpr (f + LA_AHEAD < FRAGMENTS) ring[(f + LA_AHEAD) % LA_RING] = key_fragment<CHUNKS, f + LA_AHEAD>(keys_at, key_at);
        lds_arrived<(FRAGMENTS - 1 - f < LA_AHEAD ? FRAGMENTS - 1 - f : LA_AHEAD)>(ring[f % LA_RING]);
        st[f & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ring[f % LA_RING]), qb[f >> 1], st[f & 1], 0, 0, 0);
      });
    }
    float s[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int key = kb + 8 * lq + j;
      s[j] = (row_ok && key <= pos) ? st[j >> 2][j & 3] * scale_log2 : -INFINITY;
      mx = fmaxf(mx, s[j]);
    }
    mx = max_xor32(max_xor16(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new > -INFINITY ? m_new : 0.f;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s[j] = __builtin_amdgcn_exp2f(s[j] - m_use);
      sum += s[j];
    }
    sum = sum_xor32(sum_xor16(sum));
    l_run = l_run * corr + sum;
    m_run = m_new;
    const bf16x8 pb = __builtin_bit_cast(bf16x8, uintx4{pack_two(s[0], s[1]), pack_two(s[2], s[3]), pack_two(s[4], s[5]), pack_two(s[6], s[7])});

    // O^T: this lane's eight keys of the value operand; in the tile that crosses the context's end those
    // beyond it are cleared
    const bool rescale = __builtin_amdgcn_ballot_w64(corr != 1.f) != 0;      // the whole wave: once the maxima have settled, nothing to do
    const bool crosses = kb + LA_KEYS > ctx;
    uintx4 v_mask = uintx4{~0u, ~0u, ~0u, ~0u};
    if (crosses) {
      const int vkey = kb + 8 * lq;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned int lo = vkey + 2 * w < ctx ? 0x0000ffffu : 0u;
        const unsigned int hi = vkey + 2 * w + 1 < ctx ? 0xffff0000u : 0u;
        v_mask[w] = lo | hi;
      }
    }
    {
      const unsigned int mine = values_at + value_at;
      uintx4 ring[LA_RING];
      static_for<0, LA_AHEAD>([&](auto t) { ring[t.value] = lds_read16<t.value * 1024>(mine); });
      static_for<0, DT>([&](auto tc) {
        constexpr int t = tc.value;
        if constexpr (t + LA_AHEAD < DT) ring[(t + LA_AHEAD) % LA_RING] = lds_read16<(t + LA_AHEAD) * 1024>(mine);
        if (rescale) {
#pragma unroll
          for (int i = 0; i < 4; ++i) o[t][i] *= corr;
        }
        lds_arrived<(DT - 1 - t < LA_AHEAD ? DT - 1 - t : LA_AHEAD)>(ring[t % LA_RING]);
        if (crosses) ring[t % LA_RING] &= v_mask;
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ring[t % LA_RING]), pb, o[t], 0, 0, 0);
      });
    }
  }

  if (!row_ok) return;
  const size_t global_row = (size_t)(q0 + tok) * heads + head;
  if (splits == 1) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    bf16_t* orow = out + global_row * DV + 4 * lq;
#pragma unroll
    for (int t = 0; t < DT; ++t)
      *(uintx2*)(orow + 16 * t) = uintx2{pack_two(o[t][0] * inv, o[t][1] * inv), pack_two(o[t][2] * inv, o[t][3] * inv)};
    return;
  }
  float* po = part_o + ((size_t)split * total_rows + global_row) * DV + 4 * lq;
#pragma unroll
  for (int t = 0; t < DT; ++t) *(floatx4*)(po + 16 * t) = o[t];
  if (lq == 0) {
    float* pm = part_ml + ((size_t)split * total_rows + global_row) * 2;
    pm[0] = m_run;
    pm[1] = l_run;
  }
}

// out[row] = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), m the largest m_s; the runs in order.  Block per row.
// The runs are read eight at a time with all loads of a round in flight (a run's index beyond the last reads the
// last again and is given no weight): one load after the other, each waited for, made the merge as long as
// the attention itself.
#define MERGE_ROUND 8
__global__ __launch_bounds__(128) void latent_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                           bf16_t* __restrict__ out, int splits, int total_rows, int dv) {
  const int row = blockIdx.x;
  auto stats = [&](int s) { return part_ml + ((size_t)min(s, splits - 1) * total_rows + row) * 2; };
  float top = -INFINITY;
  for (int s0 = 0; s0 < splits; s0 += MERGE_ROUND) {
    float m[MERGE_ROUND];
#pragma unroll
    for (int j = 0; j < MERGE_ROUND; ++j) m[j] = stats(s0 + j)[0];
#pragma unroll
    for (int j = 0; j < MERGE_ROUND; ++j) top = fmaxf(top, m[j]);
  }
  const float m_use = top > -INFINITY ? top : 0.f;
  float denom = 0.f;
  for (int s0 = 0; s0 < splits; s0 += MERGE_ROUND) {
    float m[MERGE_ROUND], l[MERGE_ROUND];
#pragma unroll
    for (int j = 0; j < MERGE_ROUND; ++j) {
      m[j] = stats(s0 + j)[0];
      l[j] = stats(s0 + j)[1];
    }
#pragma unroll
    for (int j = 0; j < MERGE_ROUND; ++j)
      if (s0 + j < splits) denom += l[j] * __builtin_amdgcn_exp2f(m[j] - m_use);
  }
  const float inv = denom > 0.f ? 1.f / denom : 0.f;
  for (int d = threadIdx.x; d < dv; d += 128) {
    float acc = 0.f;
    for (int s0 = 0; s0 < splits; s0 += MERGE_ROUND) {
      float m[MERGE_ROUND], o[MERGE_ROUND];
#pragma unroll
      for (int j = 0; j < MERGE_ROUND; ++j) {
        m[j] = stats(s0 + j)[0];
        o[j] = part_o[((size_t)min(s0 + j, splits - 1) * total_rows + row) * dv + d];
      }
#pragma unroll
      for (int j = 0; j < MERGE_ROUND; ++j)
        if (s0 + j < splits) acc += o[j] * __builtin_amdgcn_exp2f(m[j] - m_use);
    }
    out[(size_t)row * dv + d] = float_to_bf16(acc * inv);
  }
}

template <int DK, int DV>
static int launch_latent(const void* q, long long q_stride, const void* key_pages, const void* value_pages, void* out,
                         float* part_o, float* part_ml, const int* cu_q, const int* ctx_len, const int* block_table,
                         int table_stride, int num_seqs, int max_q_len, int heads, int block_size, int num_blocks,
                         float scale, int splits, int tokens, hipStream_t stream) {
  const long long rows = (long long)max_q_len * heads;
  const dim3 grid((unsigned)((rows + LA_ROWS - 1) / LA_ROWS), splits, num_seqs);
  constexpr int lds = 2 * (LA_KEYS * DK + DV * 32) * 2;   // two buffers of a tile's keys and its transposed values
  static bool sized = false;                              // more than 64 KB of LDS a block has to be asked for, once a kernel
  if (lds > 64 * 1024 && !sized) {
    if (hipFuncSetAttribute((const void*)latent_attention_kernel<DK, DV>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return FE_LAUNCH_FAILED;
    sized = true;
  }
  int block_shift = 0;
  while ((1 << block_shift) < block_size) ++block_shift;
  latent_attention_kernel<DK, DV><<<grid, 256, lds, stream>>>(
      (const bf16_t*)q, (size_t)q_stride, (const bf16_t*)key_pages, (const bf16_t*)value_pages, (bf16_t*)out, part_o,
      part_ml, cu_q, ctx_len, block_table, table_stride, heads, block_shift, num_blocks, scale * 1.4426950408889634f,
      splits, tokens * heads);
  if (splits > 1) latent_merge_kernel<<<tokens * heads, 128, 0, stream>>>(part_o, part_ml, (bf16_t*)out, splits, tokens * heads, DV);
  return fe_check_launch();
}

// The (DK, DV) pairs compiled below; 0 for any other.
extern "C" int fe_latent_attention_supported(int row_dim, int value_dim) {
  return (row_dim == 576 && value_dim == 512) || (row_dim == 320 && value_dim == 256) || (row_dim == 192 && value_dim == 128) ||
         (row_dim == 160 && value_dim == 128) || (row_dim == 96 && value_dim == 64);
}

extern "C" int fe_latent_attention(const void* q, long long q_stride, const void* key_pages, const void* value_pages, void* out,
                                   float* part_o, float* part_ml, const int* cu_q, const int* ctx_len,
                                   const int* block_table, int table_stride, int num_seqs, int max_q_len, int heads,
                                   int row_dim, int value_dim, int block_size, int num_blocks, float scale, int splits,
                                   int tokens, hipStream_t stream) {
  if (tokens <= 0 || num_seqs <= 0) return FE_OK;
  if (heads < 1 || max_q_len < 1 || block_size < 8 || (block_size & (block_size - 1)) || num_blocks < 1 || splits < 1 || splits > 64 ||
      num_seqs > 65535 || q_stride < (long long)heads * row_dim || q_stride % 8 || (splits > 1 && (!part_o || !part_ml)) ||
      (long long)tokens * heads > 0x7fffffffLL || !fe_latent_attention_supported(row_dim, value_dim))
    return FE_BAD_ARGUMENT;
#define CASE(DK, DV)                                                                                                   \
  if (row_dim == DK && value_dim == DV)                                                                                \
    return launch_latent<DK, DV>(q, q_stride, key_pages, value_pages, out, part_o, part_ml, cu_q, ctx_len, block_table, \
                                 table_stride, num_seqs, max_q_len, heads, block_size, num_blocks, scale, splits, tokens, stream)
  CASE(576, 512);
  CASE(320, 256);
  CASE(192, 128);
  CASE(160, 128);
  CASE(96, 64);
#undef CASE
  return FE_BAD_ARGUMENT;
}
