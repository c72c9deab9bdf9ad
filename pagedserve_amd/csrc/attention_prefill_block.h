// The tiled prefill attention's block (see attention_prefill.hip for the method): shared by the
// kernel of that file and by the kernel of attention_mixed.hip, which runs such blocks beside
// the blocks of the decode attention in one launch.
#pragma once
#include <math.h>

#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define AP_QUERIES 64      // queries per block (32 with QW = 1, 128 with QW = 4)
#define AP_TABLE_MAX 2048  // block-table entries that a tile may need
#define AP_LARGE_HEAD_DIM 64   // largest head size of the blocks of 128 queries

typedef const __attribute__((address_space(1))) void* ap_global_ptr;
typedef __attribute__((address_space(3))) void* ap_lds_ptr;

template <int PENDING>
__device__ inline void ap_wait_loads_and_sync() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PENDING) : "memory");
}

// What a block keeps in LDS: the ring of stages (the waves' states are merged in the same
// bytes at the end) and the block-table entries of its keys.  (The sizes are derived once more
// inside the block's function, which checks that they agree.)
template <int NDB, int KS, int QW, int KR>
struct PrefillLds {
  static constexpr int STAGE_BYTES = 2 * (32 * KR * KS) * (NDB * 32);
  static constexpr int FIT = (KS == 2 && QW == 2 && NDB <= 4 ? 32768 : ((KS >= 4 && QW == 2) || QW == 4 ? 65536 : 98304)) / STAGE_BYTES;
  static constexpr int STAGES = FIT >= 4 ? 4 : (FIT >= 2 ? FIT : 2);
  static constexpr int MERGE_BYTES = (QW * KS - QW) * 64 * (((NDB + 1) / 2) * 16 + 2) * 4;
  static constexpr int BYTES = STAGES * STAGE_BYTES > MERGE_BYTES ? STAGES * STAGE_BYTES : MERGE_BYTES;
  __attribute__((aligned(1024))) unsigned char stages[BYTES];
  uint32_t table[AP_TABLE_MAX];
};

// The work of one block: one head of one tile of queries.  The caller provides the block's LDS
// (the kernel below its own; a kernel that runs blocks of several kinds in one launch a share
// of what all of them need).
// head_dim / 16; waves along the keys; waves along the queries; runs of 32 keys per wave and tile
template <int NDB, int KS, int QW = 2, int KR = 1>
__device__ __forceinline__ void attention_prefill_block(
    PrefillLds<NDB, KS, QW, KR>& lds, const int head, const int tile_index,
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, bf16_t* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ cu_tokens, const int* __restrict__ kv_lens,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int page_size,
    int page_shift, int num_pages, float scale, int window) {
  constexpr int HD = NDB * 16;
  constexpr int ROW = HD * 2;                    // bytes of one key in a tile
  constexpr int CH = HD / 8;                     // 16-byte pieces per row
  constexpr int SPREAD = ROW <= 256 ? 256 / ROW : 1;   // keys that share one pass over the banks
  constexpr int WAVE_KEYS = 32 * KR;             // keys of a wave per tile
  constexpr int AP_KEYS = WAVE_KEYS * KS;        // keys per tile
  constexpr int AP_WAVES = QW * KS;
  constexpr int QUERIES = 32 * QW;               // queries per block
  static_assert(QW == 1 || QW == 2 || QW == 4, "one, two or four waves along the queries");
  static_assert(KR == 1 || KR == 2, "one or two runs of keys per wave");
  constexpr int TILE_BYTES = AP_KEYS * ROW;
  constexpr int STAGE_BYTES = 2 * TILE_BYTES;    // K tile, then V tile
  // The ring may take 96 KB; with four waves along the keys (and with blocks of 128 queries)
  // 64 KB, so that two such blocks share a compute unit: the grids that take them have up to
  // two blocks per unit, and with one block per unit half of them would wait for a second
  // round (2 x 1,024 tokens of 12 heads: 1.5 us less per launch).  The blocks of four
  // waves and 64 queries, which long prompts take by the thousand, get 32 KB at head sizes up
  // to 64, two stages: four of them then share a compute unit, four waves to a SIMD (their
  // 126 registers allow it), and what one wave waits for another fills (2 x 4,096 tokens of
  // 12 heads: 97 against 114 us with a ring of four stages and two blocks to a unit).
  constexpr int FIT = (KS == 2 && QW == 2 && NDB <= 4 ? 32768 : ((KS >= 4 && QW == 2) || QW == 4 ? 65536 : 98304)) / STAGE_BYTES;
  constexpr int STAGES = FIT >= 4 ? 4 : (FIT >= 2 ? FIT : 2);
  static_assert(NDB <= 8 || STAGES == 2, "head sizes beyond 128 rely on a ring of two stages");
  constexpr int INSTRUCTIONS = KS * KR * NDB;    // load instructions per operand and stage
  // every wave issues the same number of loads (the counter of loads in flight is per wave):
  // where they do not divide evenly the last ones are issued twice
  constexpr int PER_OPERAND = (INSTRUCTIONS + AP_WAVES - 1) / AP_WAVES;
  constexpr int LOADS = 2 * PER_OPERAND;
  constexpr int NDB32 = (NDB + 1) / 2;           // blocks of 32 head dimensions
  static_assert(LOADS * 2 < 64, "the load counter has six bits");
  // the states that the waves merge at the end lie where the stages were
  constexpr int MERGE_BYTES = (AP_WAVES - QW) * 64 * (NDB32 * 16 + 2) * 4;
  constexpr int LDS_BYTES = STAGES * STAGE_BYTES > MERGE_BYTES ? STAGES * STAGE_BYTES : MERGE_BYTES;
  static_assert(LDS_BYTES == PrefillLds<NDB, KS, QW, KR>::BYTES && STAGES == PrefillLds<NDB, KS, QW, KR>::STAGES,
                "the caller's LDS is what this function lays out");
  unsigned char (&stages)[LDS_BYTES] = lds.stages;
  uint32_t (&s_table)[AP_TABLE_MAX] = lds.table;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: scalar
  const int wave_q = wave % QW;  // which 32 queries
  const int wave_k = wave / QW;  // which run of 32 keys of every tile
  const int sub = lane & 31;     // query of this lane within the wave; key or dimension row
  const int half = lane >> 5;    // which half of a step's reduction dimension
  const int kv_head = head / (heads / kv_heads);

  // blocks start in the order of their numbers, heads fastest: the caller lists the tiles that
  // see the most keys first, so the longest blocks start first and the shortest fill the gaps
  const int item = tile_item[tile_index];
  const int q0 = tile_q0[tile_index];
  const int tok0 = cu_tokens[item];
  const int count = cu_tokens[item + 1] - tok0;
  const int start = kv_lens[item] - count;   // position of the portion's first token
  const int* table = tables + (int64_t)item * table_width;

  const int qi = q0 + wave_q * 32 + sub;
  const bool q_valid = qi < count;
  const int q_pos = q_valid ? start + qi : -1;
  const int wave_first = start + q0 + wave_q * 32;
  const int wave_last_q = q0 + wave_q * 32 + 31 < count ? q0 + wave_q * 32 + 31 : count - 1;
  const int wave_last = start + wave_last_q;
  const bool wave_active = q0 + wave_q * 32 < count;
  const int tile_last_q = q0 + QUERIES - 1 < count ? q0 + QUERIES - 1 : count - 1;
  const int key_end = start + tile_last_q + 1;
  int key_begin = 0;
  if (window > 0 && start + q0 - window + 1 > 0) key_begin = start + q0 - window + 1;

  // the block-table entries of keys key_begin .. key_end - 1
  const int first_logical = page_shift >= 0 ? (key_begin >> page_shift) : key_begin / page_size;
  const int last_logical = page_shift >= 0 ? ((key_end - 1) >> page_shift) : (key_end - 1) / page_size;
  // kept as the number of the page's first key row of this head within the pool (a row: one
  // key's HD values; the host checks that the pool has fewer than 2^32 of them), so that a
  // load's address is one multiplication away
  const uint32_t page_rows = (uint32_t)kv_heads * (uint32_t)page_size;
  const uint32_t head_rows = (uint32_t)kv_head * (uint32_t)page_size;
  for (int i = tid; i <= last_logical - first_logical && i < AP_TABLE_MAX; i += 64 * QW * KS) {
    const int logical = first_logical + i;
    int page = logical < table_width ? table[logical] : 0;
    page = (page >= 0 && page < num_pages) ? page : 0;         // never an address outside the pool
    s_table[i] = (uint32_t)page * page_rows + head_rows;
  }

  // queries as column operand of the first product: lane (query sub, dims step*16 + half*8 ..)
  bf16x8 qf[NDB];
#pragma unroll
  for (int step = 0; step < NDB; ++step) {
    const uint4 zero = {0u, 0u, 0u, 0u};
    const uint4 raw = q_valid ? *reinterpret_cast<const uint4*>(
                                    q + (int64_t)(tok0 + qi) * q_stride + (int64_t)head * HD +
                                    step * 16 + half * 8)
                              : zero;
    qf[step] = *reinterpret_cast<const bf16x8*>(&raw);
  }

  // ---- loads.  Lane l of load instruction j of an operand fills bytes j*1024 + l*16 of the
  // tile: piece (l*16 % ROW) / 16 of key (j*1024 + l*16) / ROW, which holds the key's piece
  // number (slot - key / SPREAD) mod CH.
  int load_key[PER_OPERAND], load_piece[PER_OPERAND];
#pragma unroll
  for (int j = 0; j < PER_OPERAND; ++j) {
    const int number = wave * PER_OPERAND + j < INSTRUCTIONS ? wave * PER_OPERAND + j : INSTRUCTIONS - 1;
    const int offset = number * 1024 + lane * 16;
    const int key_local = offset / ROW;
    const int slot = (offset - key_local * ROW) / 16;
    load_key[j] = key_local;
    load_piece[j] = (slot + CH - (key_local / SPREAD) % CH) % CH;
  }
  const int page_mask = page_size - 1;                // where the page size is a power of two
  auto issue = [&](int tile_number, int k0) {
    unsigned char* stage = stages + (tile_number % STAGES) * STAGE_BYTES;
    // the rows first (their table entries are then on their way together), then the loads
    uint32_t row[PER_OPERAND];
#pragma unroll
    for (int j = 0; j < PER_OPERAND; ++j) {
      // keys outside the tile's visible range are fetched from a visible key instead: they
      // are masked below, and whatever lies in pages that were given back is never read
      int key = k0 + load_key[j];
      key = key < key_begin ? key_begin : (key >= key_end ? key_end - 1 : key);
      int logical, within;
      if (page_shift >= 0) {
        logical = key >> page_shift;
        within = key & page_mask;
      } else {
        logical = key / page_size;
        within = key - logical * page_size;
      }
      row[j] = s_table[logical - first_logical] + (uint32_t)within;
    }
#pragma unroll
    for (int j = 0; j < PER_OPERAND; ++j) {
      const uint64_t offset = (uint64_t)row[j] * (uint32_t)HD + (uint32_t)(load_piece[j] * 8);
      const int number = wave * PER_OPERAND + j < INSTRUCTIONS ? wave * PER_OPERAND + j : INSTRUCTIONS - 1;
      const int dst = number * 1024;
      __builtin_amdgcn_global_load_lds((ap_global_ptr)(k_pool + offset), (ap_lds_ptr)(stage + dst),
                                       16, 0, 0);
      __builtin_amdgcn_global_load_lds((ap_global_ptr)(v_pool + offset),
                                       (ap_lds_ptr)(stage + TILE_BYTES + dst), 16, 0, 0);
    }
  };

  // Scores are kept in units of log 2 (scale * log2(e) folded into one factor), so that
  // every exponential is one v_exp_f32; probabilities are rounded to bfloat16 right after.
  const float scale_log2 = scale * 1.4426950408889634f;
  float m = -INFINITY, l = 0.f;
  f32x16 acc[NDB32];
#pragma unroll
  for (int db = 0; db < NDB32; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

  // ---- operand addresses inside a tile
  // K row operand: lane (key sub, half) reads piece 2*step + half of key sub of each of the
  // wave's runs of 32 keys
  int k_off[KR][NDB];
#pragma unroll
  for (int r = 0; r < KR; ++r) {
    const int key_local = wave_k * WAVE_KEYS + r * 32 + sub;
    const int turn = (key_local / SPREAD) % CH;
#pragma unroll
    for (int step = 0; step < NDB; ++step)
      k_off[r][step] = key_local * ROW + ((2 * step + half + turn) % CH) * 16;
  }
  // V row operand through the transposing read: in the 16 lanes of group g = lane / 16, lane r
  // points at dimensions d0 + 4 (r % 4) .. + 3 of key base + half*4 + r / 4 (+ 8 for the second
  // read) and receives dimension d0 + r of four keys, d0 = db*32 + (g & 1) * 16.
  // (a run of 32 keys is two instructions' worth of 16)
  int v_off[2 * KR][NDB32][2];
  {
    const int r16 = lane & 15;
    const int v_dim = ((lane >> 4) & 1) * 16 + 4 * (r16 & 3);        // within the block of 32 dims
    const int v_key = wave_k * WAVE_KEYS + half * 4 + (r16 >> 2);     // first 16 keys of the wave
#pragma unroll
    for (int run = 0; run < 2 * KR; ++run)
#pragma unroll
      for (int db = 0; db < NDB32; ++db) {
        int dim = db * 32 + v_dim;
        if (dim >= HD) dim -= 16;       // the padded half of the last block: any valid piece
#pragma unroll
        for (int second = 0; second < 2; ++second) {
          const int key_local = v_key + run * 16 + second * 8;
          const int slot = ((dim >> 3) + (key_local / SPREAD)) % CH;
          v_off[run][db][second] = TILE_BYTES + key_local * ROW + slot * 16 + (dim & 7) * 2;
        }
      }
  }

  const int k_first = key_begin / AP_KEYS * AP_KEYS;
  const int tiles = (key_end - k_first + AP_KEYS - 1) / AP_KEYS;
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // the table is in LDS
  // the queries have arrived with that; a use here keeps the compiler from waiting for them
  // (and with them for every tile in flight) inside the loop
#pragma unroll
  for (int step = 0; step < NDB; ++step) asm volatile("" : "+v"(qf[step]));
#pragma unroll
  for (int d = 0; d < STAGES - 1; ++d)
    if (d < tiles) issue(d, k_first + d * AP_KEYS);

  // ---- the parts of an iteration
  typedef u32x4 KeyRegs[KR][NDB];
  typedef u32x2 ValueRegs[2 * KR][NDB32][2];
  constexpr int V_READS = 4 * NDB32 * KR;
  auto wave_keys = [&](int t) { return k_first + t * AP_KEYS + wave_k * WAVE_KEYS; };
  // a wave's keys of a tile are skipped where no query of the wave can see them
  auto sees = [&](int kw) {
    return wave_active && kw <= wave_last && kw < key_end &&
           !(window > 0 && kw + WAVE_KEYS - 1 < wave_first - window + 1);
  };
  auto stage_of = [&](int t) {
    return (uint32_t)(uintptr_t)(ap_lds_ptr)stages + (uint32_t)((t % STAGES) * STAGE_BYTES);
  };
  // S^T: element e is key (e/4)*8 + half*4 + e%4 of the run.  The operand reads are written
  // as assembly: the compiler would otherwise wait for every tile in flight before each.
  auto read_keys = [&](uint32_t stage_base, KeyRegs& kr) {
#pragma unroll
    for (int r = 0; r < KR; ++r)
#pragma unroll
      for (int step = 0; step < NDB; ++step)
        asm volatile("ds_read_b128 %0, %1" : "=v"(kr[r][step]) : "v"(stage_base + k_off[r][step]) : "memory");
  };
  auto read_values = [&](uint32_t stage_base, ValueRegs& vr) {
#pragma unroll
    for (int run = 0; run < 2 * KR; ++run)
#pragma unroll
      for (int db = 0; db < NDB32; ++db)
#pragma unroll
        for (int second = 0; second < 2; ++second)
          asm volatile("ds_read_b64_tr_b16 %0, %1"
                       : "=v"(vr[run][db][second])
                       : "v"(stage_base + v_off[run][db][second])
                       : "memory");
  };
  auto scores = [&](KeyRegs& kr, f32x16 (&s)[KR]) {
#pragma unroll
    for (int r = 0; r < KR; ++r) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[r][e] = 0.f;
#pragma unroll
      for (int step = 0; step < NDB; ++step) {
        asm volatile("" : "+v"(kr[r][step]));   // used only behind the wait
        s[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&kr[r][step]),
                                                     qf[step], s[r], 0, 0, 0);
      }
    }
  };
  // softmax of a wave's scores of one tile and the second product (the values' reads may
  // still be in flight when it starts)
  auto weigh = [&](const int kw, f32x16 (&s)[KR], ValueRegs& vr) {
    // all of these keys are visible to every query of the wave: no mask
      const bool masked = kw + WAVE_KEYS - 1 > wave_first || kw + WAVE_KEYS > key_end ||
                          (window > 0 && kw < wave_last - window + 1) || !q_valid;
      // scores stay unscaled until the exponential: p = 2^(s c - m), with m kept in scaled units
      float tile_max = -INFINITY;
      if (__builtin_amdgcn_readfirstlane(__any(masked) ? 1 : 0)) {
#pragma unroll
        for (int r = 0; r < KR; ++r)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = kw + r * 32 + (e >> 2) * 8 + half * 4 + (e & 3);
            const bool visible = (key <= q_pos) & (window <= 0 || q_pos - key < window);
            s[r][e] = visible ? s[r][e] : -INFINITY;
            tile_max = fmaxf(tile_max, s[r][e]);
          }
      } else {
#pragma unroll
        for (int r = 0; r < KR; ++r)
#pragma unroll
          for (int e = 0; e < 16; ++e) tile_max = fmaxf(tile_max, s[r][e]);
      }
      tile_max = halves_max(tile_max) * scale_log2;   // scale > 0
      const float m_new = fmaxf(m, tile_max);
      // A query that has seen nothing yet (m_new = -inf) takes 0 as its reference: its scores
      // are all -inf and their exponentials 0.  Other lanes of the wave may differ, so the
      // products below run in any case.
      const float reference = (m_new == -INFINITY) ? 0.f : m_new;
      float tile_sum = 0.f;
      u32x4 p[2 * KR];      // per 16 keys
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        uint32_t words[8];
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(s[r][e], scale_log2, -reference));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(s[r][e + 1], scale_log2, -reference));
          tile_sum += p0 + p1;
          words[e >> 1] = pack2_bf16(p0, p1);
        }
        p[2 * r] = u32x4{words[0], words[1], words[2], words[3]};
        p[2 * r + 1] = u32x4{words[4], words[5], words[6], words[7]};
      }
      tile_sum = halves_sum(tile_sum);
      // the running maximum rarely moves after the first tiles: rescale only where it did
      if (__builtin_amdgcn_readfirstlane(__any(m_new != m) ? 1 : 0)) {
        const float correction = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - reference);
        l *= correction;
#pragma unroll
        for (int db = 0; db < NDB32; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[db][e] *= correction;
        m = m_new;
      }
      l += tile_sum;

      // O^T += V^T P^T, 16 keys per instruction: slots 0..3 are keys base + half*4 + 0..3,
      // slots 4..7 keys base + 8 + half*4 + 0..3, in both operands
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the values have arrived
#pragma unroll
      for (int run = 0; run < 2 * KR; ++run)
#pragma unroll
        for (int db = 0; db < NDB32; ++db) {
          asm volatile("" : "+v"(vr[run][db][0]), "+v"(vr[run][db][1]));   // used only behind the wait
          const u32x4 raw = {vr[run][db][0].x, vr[run][db][0].y, vr[run][db][1].x, vr[run][db][1].y};
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              *reinterpret_cast<const bf16x8*>(&raw), *reinterpret_cast<const bf16x8*>(&p[run]),
              acc[db], 0, 0, 0);
        }
  };

  for (int t = 0; t < tiles; ++t) {
    const int k0 = k_first + t * AP_KEYS;
    const int ahead = tiles - 1 - t < STAGES - 2 ? tiles - 1 - t : STAGES - 2;
    if (ahead <= 0) ap_wait_loads_and_sync<0>();
    else if (ahead == 1) ap_wait_loads_and_sync<LOADS>();
    else ap_wait_loads_and_sync<2 * LOADS>();
    // the stage that the tile before this one lay in is free since the barrier: the tile that
    // is STAGES - 1 ahead is asked for at once
    if (t + STAGES - 1 < tiles) issue(t + STAGES - 1, k0 + (STAGES - 1) * AP_KEYS);
    const int kw = wave_keys(t);
    if (!sees(kw)) continue;
    const uint32_t stage_base = stage_of(t);
    KeyRegs kr;
    ValueRegs vr;
    if constexpr (NDB <= 8) {
      // the transposing reads of V are issued right behind the keys'
      read_keys(stage_base, kr);
      read_values(stage_base, vr);
      // The compiler does not know that the registers read by assembly are still on their
      // way: it touches them only behind the statements that name them again, each of which
      // stands behind a wait on the same straight path.  Reads come back in the order of
      // issue: here the keys have arrived, the values may still be in flight while the scores
      // are made and weighed.
      asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(V_READS < 15 ? V_READS : 15) : "memory");
    } else {
      // Head sizes beyond 128 need more registers than a wave's 256 vector registers: the
      // compiler then moves values to the accumulation registers where it sees fit, also a
      // register that an assembly read above has not yet filled.  Here the reads are the
      // compiler's own (it waits for them itself, and for every load in flight before them,
      // which costs nothing with a ring of two stages: none is in flight at this point).
      typedef short ap_i16x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int r = 0; r < KR; ++r)
#pragma unroll
        for (int step = 0; step < NDB; ++step)
          kr[r][step] = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(
              (uintptr_t)(stage_base + k_off[r][step]));
#pragma unroll
      for (int run = 0; run < 2 * KR; ++run)
#pragma unroll
        for (int db = 0; db < NDB32; ++db)
#pragma unroll
          for (int second = 0; second < 2; ++second) {
            const ap_i16x4 raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                reinterpret_cast<__attribute__((address_space(3))) ap_i16x4*>(
                    (uintptr_t)(stage_base + v_off[run][db][second])));
            vr[run][db][second] = *reinterpret_cast<const u32x2*>(&raw);
          }
    }
    f32x16 s[KR];
    scores(kr, s);
    weigh(kw, s, vr);
  }

  // ---- the KS states of a query are merged by the wave with the first run of keys.  The
  // accumulators of waves with the same queries have the same layout, so lane meets lane.
  if (KS > 1) {
    constexpr int STATE = NDB32 * 16 + 2;      // floats per lane
    static_assert((AP_WAVES - QW) * 64 * STATE * 4 == MERGE_BYTES, "the merge reuses the stages");
    ap_wait_loads_and_sync<0>();               // every wave is past its last operand reads
    float* states = reinterpret_cast<float*>(stages);
    if (wave_k > 0) {
      float* mine = states + ((wave_k - 1) * QW + wave_q) * 64 * STATE + lane;
      mine[0] = m;
      mine[64] = l;
#pragma unroll
      for (int db = 0; db < NDB32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) mine[(2 + db * 16 + e) * 64] = acc[db][e];
    }
    __syncthreads();
    if (wave_k > 0) return;
#pragma unroll 1
    for (int other = 1; other < KS; ++other) {
      const float* theirs = states + ((other - 1) * QW + wave_q) * 64 * STATE + lane;
      const float m_o = theirs[0];
      const float l_o = theirs[64];
      const float m_n = fmaxf(m, m_o);
      const float c_mine = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_n);
      const float c_theirs = (m_o == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_o - m_n);
      l = l * c_mine + l_o * c_theirs;
      m = m_n;
#pragma unroll
      for (int db = 0; db < NDB32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          acc[db][e] = acc[db][e] * c_mine + theirs[(2 + db * 16 + e) * 64] * c_theirs;
    }
  }

  // element e of an accumulator: head dimension db*32 + (e/4)*8 + half*4 + e%4 of query `sub`
  if (q_valid && l > 0.f) {
    const float inv = 1.0f / l;
    bf16_t* dst = out + (int64_t)(tok0 + qi) * out_stride + (int64_t)head * HD;
#pragma unroll
    for (int db = 0; db < NDB32; ++db)
#pragma unroll
      for (int quad = 0; quad < 4; ++quad) {
        const int dim = db * 32 + quad * 8 + half * 4;
        if (dim >= HD) continue;
        uint2 packed;
        packed.x = pack2_bf16(acc[db][quad * 4] * inv, acc[db][quad * 4 + 1] * inv);
        packed.y = pack2_bf16(acc[db][quad * 4 + 2] * inv, acc[db][quad * 4 + 3] * inv);
        *reinterpret_cast<uint2*>(dst + dim) = packed;
      }
  }
}

template <int NDB, int KS, int QW = 2, int KR = 1>
__global__ __launch_bounds__(64 * QW * KS) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, bf16_t* __restrict__ out, int64_t out_stride,
    const int* __restrict__ tile_item, const int* __restrict__ tile_q0,
    const int* __restrict__ cu_tokens, const int* __restrict__ kv_lens,
    const int* __restrict__ tables, int table_width, int heads, int kv_heads, int page_size,
    int page_shift, int num_pages, float scale, int window) {
  __shared__ PrefillLds<NDB, KS, QW, KR> lds;
  attention_prefill_block<NDB, KS, QW, KR>(lds, blockIdx.x, blockIdx.y, q, q_stride, k_pool, v_pool, out,
                                           out_stride, tile_item, tile_q0, cu_tokens, kv_lens, tables,
                                           table_width, heads, kv_heads, page_size, page_shift,
                                           num_pages, scale, window);
}

