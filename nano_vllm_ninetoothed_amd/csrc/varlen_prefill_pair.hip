// Varlen (packed THD) causal prefill attention for gfx950, the form for grouped-query heads with an even group size:
// head_dim 128, bf16 MFMA for both products, fp32 online softmax, K/V tiles staged through LDS.  Two instantiations: keys
// that are the sequences' own tokens, and (PREFIX) keys behind a cached prefix, packed with offsets of their own or in the
// paged caches, with the causal diagonal aligned bottom-right (query row i of a sequence sees keys 0 .. i + kv_len - len).  The tile (blocks A, B, C, hand scheduled around the MFMAs) is the one of
// varlen_prefill.hip; what differs is what a wave's 32 MFMA columns are and how work reaches a workgroup.
//
// Work decomposition
//   item      = 64 query rows of one sequence x the two query heads 2u, 2u+1 (which share a kv head).  Wave w of the
//               workgroup owns rows 16w .. 16w+15; MFMA column n of the wave is (head n >> 4, row n & 15).  Both heads read
//               the same K/V tile from LDS, so the causal diagonal of an item is one 64 x 64 block instead of the 128 x 128
//               of a 128-row item: half as many tile slots are spent on keys above the diagonal.
//   launch    = resident workgroups (two per CU), each working through a list of items.  With 8 kv heads the workgroup id
//               modulo 8 (the XCD it lands on) is the kv head it serves, so an XCD's L2 holds one kv head's K/V.  Items are
//               ranked heaviest first (highest q tile first, then sequence).  A workgroup's first two items are fixed by its
//               id; every further one is drawn from a counter in device memory at the top of the item before it, and the
//               ticket has arrived by that item's last tile (an item of one tile waits for it).
//   hand-over = the K/V pipeline does not stop between items: the last tile of an item carries, in its MFMA slots, the
//               direct-to-LDS loads of the next item's first K/V tile (into the tile buffers the last tile does not use) and
//               the loads of the next item's Q operand (straight into the registers of the old one, which block A of the
//               last tile has finished with).  What is left between two items is the epilogue of the old one.
//   epilogue  = the wave's 32 columns x 128 outputs go through LDS (the buffers of the item's last tile, swizzled so that
//               writes and reads cover all banks) and leave as whole 256-byte rows.
#include "prefill_common.h"
#include <atomic>
#include <type_traits>

namespace mops {

constexpr int kPairRows = 64;          // q rows per item
constexpr int kPairWaveRows = 16;      // q rows per wave (x 2 heads = 32 MFMA columns)
constexpr int kPairMaxBatch = 512;     // sequences per launch (their offsets live in LDS)
constexpr int kPairMaxTiles = 1024;    // q tiles per sequence (65536 tokens)
constexpr int kPairTable = 1024;       // (q tile, sequence) pairs whose rank -> pair mapping is tabulated in LDS
constexpr int kPairSlots = 128;        // launches that may overlap on one device (one counter row each)
constexpr int kPairPrefixBatch = 64;   // sequences per launch of the PREFIX form
constexpr int kPairBlockEntries = 768; // block table entries (sequences x table width) the PREFIX form holds in LDS

// Item counters, one row per slot: [c] next ticket of class c (the workgroups with id % classes == c), [8] workgroups
// that have finished.  The last workgroup to finish zeroes its row, so a row is all zeros between launches.
__device__ unsigned g_pair_tickets[kPairSlots][16];

struct PairLaunch {
  int classes;          // 8 when there are 8 kv heads (class = kv head = XCD), else 1
  int units_per_class;  // head pairs per class
  int units_per_kv;     // head pairs per kv head (group / 2)
  int upc_shift;        // log2(units_per_class) when that is a power of two, else -1
  int members;          // workgroups per class
  int q_tiles;          // bound on the q tiles (64 rows) of a sequence
  int slot;             // counter row
  int table_w;          // PREFIX, paged caches: block table entries per sequence held in LDS
  int tiles_per_block;  // PREFIX, paged caches: 64-key tiles per cache block
};

// One 16-byte piece of the Q operand, loaded without the compiler knowing that the result arrives later: it then inserts
// no wait of its own (which, placed in front of the first MFMAs that read the operand, would also wait for the tile
// loads issued in between).  The operand is tied to its register on both sides, nothing reads it until the barrier at
// the top of the next item's first tile, and that barrier waits for every load of the wave.
template <int OFF>
__device__ __forceinline__ void q_piece_async(bf16x8& dst, const char* ptr) {
  asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(dst) : "v"(ptr), "n"(OFF) : "memory");
}

struct PairItem {
  int valid, seq_begin, seq_len, q0, unit, kv;   // unit: the head pair 2u, 2u + 1; kv: its kv head
  // PREFIX: the sequence's keys.  kbegin: first key row (packed) or first entry of the sequence's block table in LDS (paged);
  // kv_len: number of keys; shift = kv_len - seq_len: query row i sees keys 0 .. i + shift; steady: every cache block the
  // item looks at exists
  int kbegin, kv_len, shift, steady;
};

template <bool PREFIX>
__global__ __launch_bounds__(kPThreads, 2) void varlen_prefill_pair_kernel(const PrefillParams p, const PairLaunch L) {
  // the factor between a score as the MFMA delivers it and the base-2 exponent (the sign of a negative scale is moved into Q)
  // (never exactly zero: a masked score is -inf, and -inf * 0 would be NaN where the probability has to be 0)
  const float ec = fmaxf(fabsf(p.scale_log2), 1e-30f);
  // One array, so that the tile buffers start at the workgroup's LDS offset 0: a direct-to-LDS load takes its destination
  // from M0 as a plain offset.  K[2] then V[2] (16 KiB each), then the tables of the rank -> item mapping.
  constexpr int kTabCu = 0, kTabCnt = kPairMaxBatch + 4, kTabFrom = kTabCnt + kPairMaxBatch, kTabTicket = kTabFrom + kPairMaxTiles + 4,
                kTabPair = kTabTicket + 4, kTabCuK = kTabPair + kPairTable, kTabBlocks = kTabCuK + kPairPrefixBatch + 4,
                kTabEnd = PREFIX ? kTabBlocks + kPairBlockEntries : kTabCuK;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * kPTile + kTabEnd * 4];
  static_assert(2 * (4 * kPTile + kTabEnd * 4) <= 160 * 1024, "two workgroups per CU");
  int* const tab = reinterpret_cast<int*>(lds + 4 * kPTile);
  int* const t_cu = tab + kTabCu;        // cu_seqlens [batch + 1]
  int* const t_cnt = tab + kTabCnt;      // q tiles of sequence b
  int* const t_from = tab + kTabFrom;    // (q tile, sequence) pairs whose q tile index is >= l, l = 0 .. q_tiles + 1
  int* const t_pair = tab + kTabPair;    // pair of rank r as (sequence << 16 | q tile), when the launch is small enough for the table
  int* const t_tk = tab + kTabTicket;    // the ticket drawn during the current item
  int* const t_cuk = tab + kTabCuK;      // PREFIX: cu_seqlens_k [batch + 1]
  int* const t_bt = tab + kTabBlocks;    // PREFIX, paged: block table, table_w entries per sequence, -1 where there is no such block
  const bool paged = PREFIX && p.block_table != nullptr;
  unsigned char* const lds_k = lds;
  unsigned char* const lds_v = lds + 2 * kPKTile;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int n = lane & 31;    // MFMA column of the wave
  const int jj = lane >> 5;   // half: k slice / row-quad selector
  const int hsel = n >> 4;    // which of the unit's two heads the column belongs to
  const int rloc = n & 15;    // its row inside the wave's 16 rows

  // ---- tables of the rank -> item mapping (once per workgroup)
  // (a thread takes both offsets of its sequence from memory: the q tile counts need no second pass over LDS)
  for (int b = tid; b < ((p.batch + 15) & ~15); b += kPThreads) {
    int cnt = 0;
    if (b < p.batch) {
      const int qs = p.cu_seqlens[b], qe = p.cu_seqlens[b + 1];
      t_cu[b] = qs;
      if (b == p.batch - 1) t_cu[p.batch] = qe;
      const int len = min(qe, p.total_tokens) - qs;
      cnt = (qs >= 0 && len > 0) ? min((len + kPairRows - 1) / kPairRows, L.q_tiles) : 0;
    }
    t_cnt[b] = cnt;   // zero up to a multiple of 16: the passes below read the counts sixteen at a time
  }
  if (PREFIX) {
    for (int i = tid; i <= p.batch; i += kPThreads) t_cuk[i] = p.cu_seqlens_k[i];
    if (paged) {
      for (int i = tid; i < p.batch * L.table_w; i += kPThreads) {
        const int b = i / L.table_w;
        const int e = p.block_table[(int64_t)b * p.block_table_row_stride + (i - b * L.table_w)];
        t_bt[i] = (e >= 0 && e < p.num_blocks) ? e : -1;
      }
    }
  }
  __syncthreads();
  // Small launches also tabulate rank -> pair, a lookup per item instead of two searches: the thread that works out
  // from[l] knows where the pairs of q tile l - 1 start (at rank from[l]) and writes them down, sequences in order.
  const bool may_tabulate = p.batch <= 64 && (p.total_tokens >> 6) + p.batch <= kPairTable;
  typedef int i32x4 __attribute__((ext_vector_type(4)));
  const i32x4* const cnt4 = reinterpret_cast<const i32x4*>(t_cnt);
  for (int l = tid; l <= L.q_tiles + 1; l += kPThreads) {
    int s = 0;
    if (l < L.q_tiles)
      for (int b = 0; b < p.batch; b += 16) {
        const i32x4 c0 = cnt4[b >> 2], c1 = cnt4[(b >> 2) + 1], c2 = cnt4[(b >> 2) + 2], c3 = cnt4[(b >> 2) + 3];
#pragma unroll
        for (int e = 0; e < 4; ++e) s += max(0, c0[e] - l) + max(0, c1[e] - l) + max(0, c2[e] - l) + max(0, c3[e] - l);
      }
    t_from[l] = s;
    if (may_tabulate && l >= 1 && l <= L.q_tiles) {
      for (int b = 0; b < p.batch; b += 16) {
        const i32x4 c[4] = {cnt4[b >> 2], cnt4[(b >> 2) + 1], cnt4[(b >> 2) + 2], cnt4[(b >> 2) + 3]};
#pragma unroll
        for (int e = 0; e < 16; ++e)
          if (c[e >> 2][e & 3] > l - 1) {
            if (s < kPairTable) t_pair[s] = ((b + e) << 16) | (l - 1);
            ++s;
          }
      }
    }
  }
  __syncthreads();
  const int home = (int)blockIdx.x % L.classes;   // the class this workgroup serves first
  const int member = (int)blockIdx.x / L.classes;
  const int n_pairs = __builtin_amdgcn_readfirstlane(t_from[0]);
  // (offsets that are not non-decreasing can describe more pairs than the tokens allow for; the table is then not used)
  const bool tabulated = may_tabulate && n_pairs <= kPairTable;
  const int n_items = n_pairs * L.units_per_class;   // items of a class (the same for all)
  if (tid == 0) t_tk[2] = home;

  // rank (within the class, heaviest first) -> item.  Every wave works it out for itself; all values are wave-uniform.
  auto map_item = [&](int cls, int R) -> PairItem {
    PairItem it = {0, 0, 0, 0, 0, 0, 0, 0, 0, 1};
    if (R >= n_items) return it;
    // rank of the (q tile, sequence) pair and the head pair inside the class (no division for 1, 2, 4 .. pairs per class)
    const int pr = L.upc_shift >= 0 ? R >> L.upc_shift : R / L.units_per_class;
    const int unit = cls * L.units_per_class + (R - pr * L.units_per_class);
    int m, b = -1;
    if (tabulated) {
      const int e = t_pair[pr];
      m = e & 0xffff;
      b = e >> 16;
    } else {
    // the pair's q tile index m: the largest l with from[l] > pr; from[] is non-increasing, two levels of 64-way search
    const int S = (L.q_tiles + 64) >> 6;
    int ln = lane;
    asm volatile("" : "+v"(ln));   // opaque: keeps the compiler from holding the LDS addresses of the searches in registers for the whole kernel
    const int i1 = ln * S;
    const int v1 = i1 <= L.q_tiles ? t_from[i1] : 0;
    const unsigned long long m1 = __ballot(v1 > pr);
    if (m1 == 0) return it;
    m = (63 - __builtin_clzll(m1)) * S;
    if (S > 1) {
      const int i2 = m + ln;
      const int v2 = (ln < S && i2 <= L.q_tiles) ? t_from[i2] : 0;
      const unsigned long long m2 = __ballot(v2 > pr);
      m += 63 - __builtin_clzll(m2 | 1ull);
    }
    int r = pr - t_from[m + 1];   // rank among the sequences that have q tile m
    for (int j = 0; 64 * j < p.batch && b < 0; ++j) {
      const int bb = ln + 64 * j;
      const bool has = bb < p.batch && t_cnt[bb] > m;
      const unsigned long long mask = __ballot(has);
      const int c = __popcll(mask);
      if (r < c) {
        const int before = __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
        const unsigned long long hit = __ballot(has && before == r);
        b = 64 * j + __builtin_ctzll(hit | (1ull << 63));
      } else {
        r -= c;
      }
    }
    }
    if (b < 0) return it;
    const int seq_begin = t_cu[b];
    const int seq_len = min(t_cu[b + 1], p.total_tokens) - seq_begin;
    // q tiles are aligned to the END of the sequence: tile m covers rows [q0, q0 + 64) with q0 = len - 64 * (tiles - m), so
    // the partial tile is the first one (rows below 0 do not exist), which looks at one K/V tile, and not the last one
    const int seq_tiles = (seq_len + kPairRows - 1) / kPairRows;
    it.valid = 1;
    it.seq_begin = __builtin_amdgcn_readfirstlane(seq_begin);
    it.seq_len = __builtin_amdgcn_readfirstlane(seq_len);
    it.q0 = __builtin_amdgcn_readfirstlane(seq_len - (seq_tiles - m) * kPairRows);
    it.unit = __builtin_amdgcn_readfirstlane(unit);
    it.kv = L.classes == 8 ? cls : it.unit / L.units_per_kv;
    if (PREFIX) {
      const int kb = t_cuk[b];
      int kv_len = t_cuk[b + 1] - kb;
      kv_len = min(kv_len, paged ? L.table_w * p.block_size : p.total_k_tokens - kb);
      kv_len = kb >= 0 ? max(kv_len, 0) : 0;
      it.kv_len = __builtin_amdgcn_readfirstlane(kv_len);
      it.shift = it.kv_len - it.seq_len;
      it.kbegin = __builtin_amdgcn_readfirstlane(paged ? b * L.table_w : kb);
      if (paged) {
        // whether every block under the keys the item looks at exists
        const int kv_end = max(0, min(it.kv_len, it.q0 + kPairRows + it.shift));
        const int used = (kv_end + p.block_size - 1) / p.block_size;
        int ln = lane;
        asm volatile("" : "+v"(ln));
        bool bad = false;
        for (int j = 0; j < used; j += 64) bad |= (j + ln < used) && t_bt[it.kbegin + j + ln] < 0;
        it.steady = __ballot(bad) == 0;
      }
    }
    return it;
  };

  // ---- cooperative tile loads, HBM -> LDS without a stop in registers (global_load_lds_dwordx4: the 64 lanes of a wave
  //      deposit 64 x 16 bytes at consecutive LDS addresses).  Instruction i of wave w brings rows 16i + 4w .. + 3 of the
  //      tile: lane (rr = lane >> 4, pos = lane & 15) fills 16-byte position `pos` of row 16i + 4w + rr.  LDS rows are
  //      unpadded; position pos of K row r holds piece pos ^ (r & 15), of V row r piece pos ^ 4 * (r & 3), so that the K
  //      operand read and the transposing V read each cover all banks.  Rows past the end of the sequence read the
  //      sequence's last row (finite data; their scores are masked, their probabilities zero).
  const int ld_row = tid >> 4;     // 4 * wave + rr
  const int ld_pos = tid & 15;
  const unsigned k_row_bytes = (unsigned)(p.k_ts * 2), v_row_bytes = (unsigned)(p.v_ts * 2);
  const unsigned kswz = (unsigned)((ld_pos ^ ld_row) << 4), vswz = (unsigned)((ld_pos ^ ((ld_row & 3) << 2)) << 4);
  unsigned ko[4], vo[4];   // this lane's byte offsets of its pieces from a tile's base (the kv head is part of the base)
  auto set_offsets = [&](int last) {   // last: last row of the tile that exists (63 for a whole tile)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned row = (unsigned)min(ld_row + 16 * i, last);
      ko[i] = row * k_row_bytes + kswz;
      vo[i] = row * v_row_bytes + vswz;
    }
  };
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;
  // The tile's base address and the wave's LDS destination are scalar values, the lane's offset a vector register.
  // M0 carries the wave's LDS destination; lane l deposits its 16 bytes at M0 + 16 * l.  Inline assembly on purpose:
  // through the compiler's builtin every later LDS read waits for the load to land.
  auto to_lds_s = [&](uint64_t sbase, unsigned voff, unsigned lds_s) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 : : "v"(voff), "s"(sbase), "s"(lds_s) : "memory", "m0");
  };
  // a wave-uniform value the compiler holds in a vector register, moved to a scalar one, with the wait states a
  // v_readfirstlane needs behind the VALU write of its source and a memory instruction behind the write of a scalar base
  auto to_scalar = [&](unsigned v) -> unsigned {
    unsigned s_;
    asm volatile("s_nop 1\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(s_) : "v"(v));
    return s_;
  };
  const unsigned lds_s = to_scalar((unsigned)(uintptr_t)(lds_ptr_t)lds + ((unsigned)(tid >> 6) << 10));
  // the eight loads of one tile in a burst (a wave that computes nothing on the tile)
  auto loads_only = [&](uint64_t kbase, uint64_t vbase, unsigned lds_next) {
#pragma unroll
    for (int j = 0; j < 4; ++j) to_lds_s(kbase, ko[j], lds_next + (unsigned)(4 * kPKChunk * j));
#pragma unroll
    for (int j = 0; j < 4; ++j) to_lds_s(vbase, vo[j], lds_next + (unsigned)(2 * kPKTile + 4 * kPKChunk * j));
  };

  // K operand read: lane (n, jj) reads piece jj + 2 * k8 of row n (+ 32): at position (jj + 2 * k8) ^ (n & 15)
  int rd_k[8];
#pragma unroll
  for (int k8 = 0; k8 < 8; ++k8) rd_k[k8] = n * kPRow + (((jj + 2 * k8) ^ (n & 15)) << 4);
  // transposing V read: 16-lane group (d half, jj); lane addresses token row 4 * jj + rr2 of a 4-row set and 8 bytes of
  // the group's 32-byte window; the 64-byte block dt of the row sits at block dt ^ rr2
  int rd_v[4];
  {
    const int rr2 = (lane >> 2) & 3;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
      rd_v[dt] = (4 * jj + rr2) * kPRow + (((lane >> 4) & 1) << 5) + ((lane & 3) << 3) + 64 * (dt ^ rr2);
  }

  // ---- per-item state
  bf16x8 qb[8];   // Q^T as B operand: lane (n, jj) holds Q[row][head][16*kb + 8*jj .. +8) for kb = 0..7
  f32x16 acc[4];
  f32x16 s_init;  // the accumulator every score product starts from: minus the softmax reference
  float m_run, l_run;
  const int64_t q_row_bytes = p.q_ts * 2;
  // address of this lane's first Q piece of an item; rows outside the sequence take a copy of a valid row (columns are
  // independent and theirs are never stored)
  auto q_address = [&](const PairItem& it) -> const char* {
    const int row = min(max(it.q0 + kPairWaveRows * wave + rloc, 0), it.seq_len - 1);
    return reinterpret_cast<const char*>(p.q) + (int64_t)(it.seq_begin + row) * q_row_bytes + (int64_t)((2 * it.unit + hsel) * kPD + 8 * jj) * 2;
  };
  auto q_load = [&](int kb, const char* ptr) {
    switch (kb) {
      case 0: q_piece_async<0>(qb[0], ptr); break;
      case 1: q_piece_async<32>(qb[1], ptr); break;
      case 2: q_piece_async<64>(qb[2], ptr); break;
      case 3: q_piece_async<96>(qb[3], ptr); break;
      case 4: q_piece_async<128>(qb[4], ptr); break;
      case 5: q_piece_async<160>(qb[5], ptr); break;
      case 6: q_piece_async<192>(qb[6], ptr); break;
      default: q_piece_async<224>(qb[7], ptr); break;
    }
  };
  // Base addresses of an item's first K/V tile, and whether that tile holds a key the item looks at.  A tile that does
  // not (no keys at all, a cache block that does not exist) is loaded from the start of the buffer, which is memory that
  // exists, and not computed on.  PREFIX: k_ts / v_ts are the row strides of the keys, packed or inside a cache block.
  const uint64_t block_bytes = PREFIX ? (uint64_t)p.block_size * (uint64_t)p.k_ts * 2u : 0u;
  auto first_tile = [&](const PairItem& it, uint64_t& kb, uint64_t& vb) -> bool {
    const uint64_t kroot = reinterpret_cast<uint64_t>(p.k) + (uint64_t)(it.kv * kPD * 2);
    const uint64_t vroot = reinterpret_cast<uint64_t>(p.v) + (uint64_t)(it.kv * kPD * 2);
    if (!PREFIX) {
      kb = kroot + (uint64_t)((int64_t)it.seq_begin * p.k_ts * 2);
      vb = vroot + (uint64_t)((int64_t)it.seq_begin * p.v_ts * 2);
      return true;
    }
    bool ex = min(it.kv_len, it.q0 + kPairRows + it.shift) > 0;
    if (paged) {
      const int e = ex ? __builtin_amdgcn_readfirstlane(t_bt[it.kbegin]) : -1;
      ex = e >= 0;
      kb = kroot + (uint64_t)max(e, 0) * block_bytes;
      vb = vroot + (uint64_t)max(e, 0) * block_bytes;
    } else {
      kb = kroot + (uint64_t)((int64_t)(ex ? it.kbegin : 0) * p.k_ts * 2);
      vb = vroot + (uint64_t)((int64_t)(ex ? it.kbegin : 0) * p.v_ts * 2);
    }
    return ex;
  };

  // One tile, hand scheduled.  Every MFMA opens a slot; the instructions that follow it up to the next
  // scheduling fence are what the wave issues while that MFMA runs.
  //   block A: S^T = K . Q^T, the eight direct-to-LDS loads of the next tile ride in its slots
  //   block B: row max, whether the reference has to move, the first ten exponentials
  //   block C: O^T += V^T . P^T, the remaining exponentials, the row sums and the bf16 packing ride in its slots; on an
  //            item's last tile (`last`) also the eight loads of the next item's Q operand, into qb, which block A is done with
  // `horizon`: last key (sequence-relative) this lane's row may see; only read on the masked variant.
  auto tile_compute = [&](int tile, int buf, uint64_t kbase, uint64_t vbase, auto masked, auto last, int horizon, const char* qnext) {
    const unsigned lds_next = lds_s + (unsigned)((buf ^ 1) * kPKTile);
    f32x16 s[2];
    {
      const unsigned char* kt = lds_k + buf * kPKTile;
      u32x4 ka[16];
      auto rd = [&](int i) { ka[i] = *reinterpret_cast<const u32x4*>(kt + rd_k[i >> 1] + (i & 1) * 32 * kPRow); };
      for (int i0 = 0; i0 < kPAhead; ++i0) rd(i0);
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        s[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[i]), qb[i >> 1], i < 2 ? s_init : s[i & 1], 0, 0, 0);
        if (i + kPAhead < 16) rd(i + kPAhead);
        if (i & 1) {
          const int j = i >> 1;
          if (j < 4) to_lds_s(kbase, ko[j], lds_next + (unsigned)(4 * kPKChunk * j));
          else to_lds_s(vbase, vo[j - 4], lds_next + (unsigned)(2 * kPKTile + 4 * kPKChunk * (j - 4)));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    // block B
    if (decltype(masked)::value) {
      const int j0 = tile * kPBN;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = j0 + 32 * tt + 8 * (r >> 2) + 4 * jj + (r & 3);
          s[tt][r] = key <= horizon ? s[tt][r] : -INFINITY;
        }
    }
    // A wave issues in order and a dependent VALU instruction waits ~20 cycles for its operand, so the
    // softmax is written for instruction-level parallelism: four max chains, and the exponent pipeline
    // E (exp2) -> P (row sum, bf16 pack) is skewed by one MFMA slot per stage.
    float mx[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) mx[c] = max3(s[c >> 1][8 * (c & 1)], s[c >> 1][8 * (c & 1) + 1], s[c >> 1][8 * (c & 1) + 2]);
#pragma unroll
    for (int c = 0; c < 4; ++c) mx[c] = max3(mx[c], s[c >> 1][8 * (c & 1) + 3], s[c >> 1][8 * (c & 1) + 4]);
#pragma unroll
    for (int c = 0; c < 4; ++c) mx[c] = max3(mx[c], s[c >> 1][8 * (c & 1) + 5], s[c >> 1][8 * (c & 1) + 6]);
    const float m01 = max3(mx[0], mx[1], s[0][7]), m23 = max3(mx[2], mx[3], s[0][15]);
    const float m_loc = half_swap_max(max3(m01, m23, fmaxf(s[1][7], s[1][15])));
    // m_loc is relative to the reference the scores were computed against.  The reference only moves when a row's
    // maximum outgrows it by kLazyLog2 (probabilities then reach at most 2^kLazyLog2, harmless in bf16 and in the fp32
    // sums; the final division by the row sum is exact for any reference).
    float alpha = 1.0f;
    const float m_old_safe = (m_run == -INFINITY) ? 0.f : m_run;
    const float m_abs = m_loc + m_old_safe;
    const bool grow = m_abs * ec > m_run * ec + kLazyLog2;   // -inf reference: any finite maximum
    if (__any(grow)) {
      const float m_new = grow ? m_abs : m_run;
      const float m_new_safe = (m_new == -INFINITY) ? 0.f : m_new;
      alpha = __builtin_amdgcn_exp2f((m_run - m_new_safe) * ec);
      const float delta = m_new_safe - m_old_safe;   // 0 in lanes whose reference stays
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[tt][r] -= delta;
      m_run = m_new;
#pragma unroll
      for (int r = 0; r < 16; ++r) s_init[r] = -m_new_safe;
    }
    u32x4 pw[4];   // P^T as B operand for the four 16-token k blocks
    float ps0 = 0.f, ps1 = 0.f;
    float f0[16], f1[16];
    auto stage_e = [&](int q) {
      const int tt = q >> 3, r = 2 * (q & 7);
      f0[q] = __builtin_amdgcn_exp2f(s[tt][r] * ec);
      f1[q] = __builtin_amdgcn_exp2f(s[tt][r + 1] * ec);
    };
    auto stage_p = [&](int q) {
      const int tt = q >> 3, r = 2 * (q & 7);
      if (q & 1) ps1 += f0[q] + f1[q]; else ps0 += f0[q] + f1[q];
      pw[2 * tt + (r >> 3)][(r & 7) >> 1] = pack_bf16x2(f0[q], f1[q]);
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 5; ++q) stage_e(q);
    __builtin_amdgcn_sched_barrier(0);
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) acc[dt] *= alpha;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) stage_p(q);
    // block C
    {
      const unsigned char* vt = lds_v + buf * kPTile;
      s16x4 vlo[16], vhi[16];
      auto rd = [&](int i) {
        const int kb2 = i >> 2, dt = i & 3;
        vlo[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vt + rd_v[dt] + 16 * kb2 * kPRow));
        vhi[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vt + rd_v[dt] + (16 * kb2 + 8) * kPRow));
      };
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      for (int i0 = 0; i0 < kPAhead; ++i0) rd(i0);
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const s16x8 a8 = __builtin_shufflevector(vlo[i], vhi[i], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a8), __builtin_bit_cast(bf16x8, pw[i >> 2]), acc[i & 3], 0, 0, 0);
        if (i + kPAhead < 16) rd(i + kPAhead);
        // slot i finishes pair i + 4 (needed from slot 4 * ((i + 4) / 4) on) and exponentiates pair i + 5
        if (i + 4 < 16) stage_p(i + 4);
        if (i + 5 < 16) stage_e(i + 5);
        if (decltype(last)::value && (i & 1)) q_load(i >> 1, qnext);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    l_run = l_run * alpha + (ps0 + ps1);
  };

  // The same for a tile of which no row of this wave sees more than the first 32 keys: the fully masked half is neither
  // multiplied nor exponentiated.  Eight MFMAs per block.
  auto tile_compute_half = [&](int tile, int buf, uint64_t kbase, uint64_t vbase, auto last, int horizon, const char* qnext) {
    const unsigned lds_next = lds_s + (unsigned)((buf ^ 1) * kPKTile);
    f32x16 s0;
    {
      const unsigned char* kt = lds_k + buf * kPKTile;
      u32x4 ka[8];
      auto rd = [&](int i) { ka[i] = *reinterpret_cast<const u32x4*>(kt + rd_k[i]); };
      for (int i0 = 0; i0 < kPAhead; ++i0) rd(i0);
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[i]), qb[i], i == 0 ? s_init : s0, 0, 0, 0);
        if (i + kPAhead < 8) rd(i + kPAhead);
        if (i < 4) to_lds_s(kbase, ko[i], lds_next + (unsigned)(4 * kPKChunk * i));
        else to_lds_s(vbase, vo[i - 4], lds_next + (unsigned)(2 * kPKTile + 4 * kPKChunk * (i - 4)));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    {
      const int j0 = tile * kPBN;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = j0 + 8 * (r >> 2) + 4 * jj + (r & 3);
        s0[r] = key <= horizon ? s0[r] : -INFINITY;
      }
    }
    float mx[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) mx[c] = max3(s0[8 * c], s0[8 * c + 1], s0[8 * c + 2]);
#pragma unroll
    for (int c = 0; c < 2; ++c) mx[c] = max3(mx[c], s0[8 * c + 3], s0[8 * c + 4]);
#pragma unroll
    for (int c = 0; c < 2; ++c) mx[c] = max3(mx[c], s0[8 * c + 5], s0[8 * c + 6]);
    const float m_loc = half_swap_max(max3(mx[0], mx[1], fmaxf(s0[7], s0[15])));
    float alpha = 1.0f;
    const float m_old_safe = (m_run == -INFINITY) ? 0.f : m_run;
    const float m_abs = m_loc + m_old_safe;
    const bool grow = m_abs * ec > m_run * ec + kLazyLog2;
    if (__any(grow)) {
      const float m_new = grow ? m_abs : m_run;
      const float m_new_safe = (m_new == -INFINITY) ? 0.f : m_new;
      alpha = __builtin_amdgcn_exp2f((m_run - m_new_safe) * ec);
      const float delta = m_new_safe - m_old_safe;
#pragma unroll
      for (int r = 0; r < 16; ++r) s0[r] -= delta;
      m_run = m_new;
#pragma unroll
      for (int r = 0; r < 16; ++r) s_init[r] = -m_new_safe;
    }
    u32x4 pw[2];
    float ps0 = 0.f, ps1 = 0.f;
    float f0[8], f1[8];
    auto stage_e = [&](int q) {
      f0[q] = __builtin_amdgcn_exp2f(s0[2 * q] * ec);
      f1[q] = __builtin_amdgcn_exp2f(s0[2 * q + 1] * ec);
    };
    auto stage_p = [&](int q) {
      const int r = 2 * q;
      if (q & 1) ps1 += f0[q] + f1[q]; else ps0 += f0[q] + f1[q];
      pw[r >> 3][(r & 7) >> 1] = pack_bf16x2(f0[q], f1[q]);
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 5; ++q) stage_e(q);
    __builtin_amdgcn_sched_barrier(0);
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) acc[dt] *= alpha;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) stage_p(q);
    {
      const unsigned char* vt = lds_v + buf * kPTile;
      s16x4 vlo[8], vhi[8];
      auto rd = [&](int i) {
        const int kb2 = i >> 2, dt = i & 3;
        vlo[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vt + rd_v[dt] + 16 * kb2 * kPRow));
        vhi[i] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vt + rd_v[dt] + (16 * kb2 + 8) * kPRow));
      };
      typedef short s16x8 __attribute__((ext_vector_type(8)));
      for (int i0 = 0; i0 < kPAhead; ++i0) rd(i0);
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const s16x8 a8 = __builtin_shufflevector(vlo[i], vhi[i], 0, 1, 2, 3, 4, 5, 6, 7);
        acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a8), __builtin_bit_cast(bf16x8, pw[i >> 2]), acc[i & 3], 0, 0, 0);
        if (i + kPAhead < 8) rd(i + kPAhead);
        if (i + 4 < 8) stage_p(i + 4);
        if (i + 5 < 8) stage_e(i + 5);
        if (decltype(last)::value) q_load(i, qnext);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    l_run = l_run * alpha + (ps0 + ps1);
  };

  // ---- the workgroup's first two items; the first one's Q operand and first K/V tile
  //      (ranks j and 2 * members - 1 - j: the heaviest first item goes with the lightest second one)
  PairItem cur = map_item(home, member);
  PairItem nxt = map_item(home, 2 * L.members - 1 - member);
  bool draw = false;   // whether the item after the current one is drawn from the counter (every item but the first two)
  unsigned* const tickets = g_pair_tickets[L.slot];
  const uint64_t kstep = (uint64_t)kPBN * (uint64_t)p.k_ts * 2u, vstep = (uint64_t)kPBN * (uint64_t)p.v_ts * 2u;
  int clamp = 63;     // the last-row clamp ko / vo are set for
  int buf = 0;        // tile buffer pair the tile about to be computed sits in
  bool tile_exists = true;   // PREFIX: whether the tile about to be computed holds keys (see first_tile)
  if (cur.valid) {
    clamp = max(0, min(63, (PREFIX ? cur.kv_len : cur.seq_len) - 1));
    set_offsets(clamp);
    uint64_t kb0, vb0;
    tile_exists = first_tile(cur, kb0, vb0);
    loads_only(kb0, vb0, lds_s);
    const char* qa = q_address(cur);
#pragma unroll
    for (int kb = 0; kb < 8; ++kb) q_load(kb, qa);
  }

  unsigned tk = 0;   // thread 0: the ticket in flight
  // The XCDs of a device do not run at one speed (their matrix throughput under this kernel differs by several percent), so
  // a class served only by "its" workgroups finishes when its XCD does.  Lanes 0..7 of wave 0 therefore look at all the
  // class counters once per item; when the home class is ahead of the class that has got least far by kStealLead tickets,
  // the next draw is made from that class (its K/V then come through another XCD's L2: slower per tile, but work that
  // the slowest XCD no longer has to do).  Towards the end of a class's list nothing is taken from it any more, so that
  // every class ends on its own workgroups, by then at about the same time.
  constexpr int kStealLead = 8;
  unsigned snap = 0;      // wave 0, lane c: counter of class c as it was at the top of the current item
  // t_tk[0]: the ticket; t_tk[1]: the class it was drawn from; t_tk[2]: the class the next draw is made from (kept in LDS:
  // only wave 0 needs them, and the kernel has no registers to spare)
  const bool balance = L.classes == 8 && (member & 15) == 0;
  auto park_ticket = [&]() {   // wave 0, behind a barrier that has waited for the draw and the counter snapshot
    if (tid == 0) t_tk[0] = (int)tk;
    if (balance) {
      int least = 0x7fffffff, who = home;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int v = (int)__builtin_amdgcn_readlane(snap, c);
        if (v < least) {
          least = v;
          who = c;
        }
      }
      const int own = (int)__builtin_amdgcn_readlane(snap, home);
      if (tid == 0) t_tk[2] = (own >= least + kStealLead && least + 3 * L.members < n_items) ? who : home;
    }
  };
  // The barrier at the top of a tile, followed by a use of the ticket register: the barrier has waited for every memory
  // operation of the wave, the atomic included, and the (empty) use tells the compiler so; otherwise it would wait for the
  // atomic's result where the register is next written, at the top of the next item, and for everything issued before it.
  auto item_barrier = [&]() {
    tile_barrier();
    asm volatile("" : : "v"(tk));
  };
  // Whether the wave's last eight vector-memory instructions before the top of this item were the eight output stores of
  // the previous item (every row of the wave existed; else the stores are predicated and may be skipped).  The item's first
  // barrier then waits for everything but those stores: the loads of the item's first tile and of its Q operand are older,
  // memory operations complete in order, and the acknowledgement of a store is nothing the item needs.
  bool stores8 = false;
  while (cur.valid) {
    if (p.scale_log2 < 0.f) {   // the sign of a negative scale moves into Q; the operand has to have arrived for that
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(qb[0]), "+v"(qb[1]), "+v"(qb[2]), "+v"(qb[3]), "+v"(qb[4]), "+v"(qb[5]), "+v"(qb[6]), "+v"(qb[7]));
#pragma unroll
      for (int kb = 0; kb < 8; ++kb) qb[kb] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, qb[kb]) ^ 0x80008000u);   // -Q, exactly
    }
    // The ticket of the item after next; thread 0 parks it in LDS behind the item's first barrier.  A wrapping increment
    // and not an addition: the compiler turns a uniform atomic addition into one lane's addition plus a broadcast of the
    // result, which would wait for the result right here.
    if (tid < 64 && draw) {
      if (tid == 0) {
        const int target = t_tk[2];
        tk = atomicInc(&tickets[target], 0xffffffffu);
        t_tk[1] = target;
      }
      if (balance && tid < 8) snap = __hip_atomic_load(&tickets[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) s_init[r] = 0.f;
    m_run = -INFINITY;
    l_run = 0.f;

    // query row i sees keys 0 .. i + shift, of kv_len keys (shift = 0 and kv_len = seq_len without a cached prefix)
    const int shift = PREFIX ? cur.shift : 0;
    const int kv_len = PREFIX ? cur.kv_len : cur.seq_len;
    // K/V tiles the item looks at (keys 0 .. q0 + 63 + shift); an item that sees no key at all goes through one tile that
    // nobody computes on
    const int ntiles = PREFIX ? max(1, (min(kv_len, cur.q0 + kPairRows + shift) + kPBN - 1) / kPBN) : (cur.q0 + kPairRows + kPBN - 1) / kPBN;
    const int wave_row0 = cur.q0 + kPairWaveRows * wave;           // first q row (sequence-relative) of this wave
    const int my_row = wave_row0 + rloc;
    const int wave_last = wave_row0 + kPairWaveRows - 1 + shift;   // last key the wave's last row sees
    // tiles this wave has to look at, and those of them that lie wholly below its first row's diagonal
    const int my_tiles = wave_last >= 0 ? min(ntiles, wave_last / kPBN + 1) : 0;
    const int unmasked = wave_row0 + shift >= 0 ? (wave_row0 + shift + 1) / kPBN : 0;
    uint64_t kbase, vbase;   // base of the tile after the one being computed
    first_tile(cur, kbase, vbase);
    // paged caches: block and tile inside the block of the tile kbase / vbase point at; whether that tile exists
    int blk_i = 0, in_blk = 0;
    bool next_exists = tile_exists;   // tiles of one block exist together
    auto advance = [&]() {
      if (paged) {
        if (++in_blk == L.tiles_per_block) {
          in_blk = 0;
          ++blk_i;
          const int e = __builtin_amdgcn_readfirstlane(t_bt[cur.kbegin + blk_i]);
          next_exists = e >= 0;
          const uint64_t off = (uint64_t)max(e, 0) * block_bytes + (uint64_t)(cur.kv * kPD * 2);
          kbase = reinterpret_cast<uint64_t>(p.k) + off;
          vbase = reinterpret_cast<uint64_t>(p.v) + off;
          return;
        }
      }
      kbase += kstep;
      vbase += vstep;
    };
    // The item's first barrier.  (Wave 0 has one or two more operations in flight, the draw and the look at the counters; eight
    // may stay in flight there too, which then makes it wait for as many stores.)  The ticket goes to LDS behind a barrier that has waited for the draw:
    // the second one, or, for items of one or two tiles, here, where the compiler puts the wait in front of the write.
    if (stores8) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else tile_barrier();
    if (ntiles <= 2 && tid < 64 && draw) park_ticket();
    int tile = 0;
    // Steady prefix: tiles that lie below the diagonal of every wave of the item and whose successor is a whole tile (all
    // but the item's last two).  Per tile two scalar additions, the tile, the barrier.
    const int n_steady = (PREFIX && !cur.steady) ? 0 : min(ntiles - 2, cur.q0 + shift >= 0 ? (cur.q0 + shift + 1) / kPBN : 0);
    for (; tile < n_steady; ++tile) {
      advance();
      tile_compute(tile, buf, kbase, vbase, std::false_type{}, std::false_type{}, 0, nullptr);
      buf ^= 1;
      item_barrier();   // the top of the next tile
      if (tile == 0 && tid < 64 && draw) park_ticket();   // n_steady > 0 means more than two tiles
    }
    for (; tile < ntiles - 1; ++tile) {
      advance();
      // the successor is a tile of this item; only the item's last tile can reach past the end of the keys
      const int want = min(63, kv_len - 1 - (tile + 1) * kPBN);
      if (want != clamp) {
        clamp = want;
        set_offsets(clamp);
      }
      if (tile >= my_tiles || (PREFIX && !tile_exists)) loads_only(kbase, vbase, lds_s + (unsigned)((buf ^ 1) * kPKTile));
      else if (tile < unmasked) tile_compute(tile, buf, kbase, vbase, std::false_type{}, std::false_type{}, 0, nullptr);
      else if (wave_last < tile * kPBN + 32) tile_compute_half(tile, buf, kbase, vbase, std::false_type{}, my_row + shift, nullptr);
      else tile_compute(tile, buf, kbase, vbase, std::true_type{}, std::false_type{}, my_row + shift, nullptr);
      if (PREFIX) tile_exists = next_exists;
      buf ^= 1;
      item_barrier();   // the top of the next tile
      if (tile == 0 && ntiles > 2 && tid < 64 && draw) park_ticket();
    }
    // the item's last tile: its successor is the next item's first tile, and the next item's Q operand comes with it.
    // Without a next item the loads are repeated on this item's own first tile and rows (harmless, never read).
    {
      if (draw) {
        // The ticket drawn at the top of the item went to LDS one barrier ago at the latest; an item of a single tile has
        // come through one barrier only and holds another one here.
        if (ntiles == 1) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        nxt = map_item(__builtin_amdgcn_readfirstlane(t_tk[1]), 2 * L.members + __builtin_amdgcn_readfirstlane(t_tk[0]));
      }
      const PairItem& to = nxt.valid ? nxt : cur;
      next_exists = first_tile(to, kbase, vbase);
      const int want = max(0, min(63, (PREFIX ? to.kv_len : to.seq_len) - 1));
      if (want != clamp) {
        clamp = want;
        set_offsets(clamp);
      }
      const char* qnext = q_address(to);
      if (tile >= my_tiles || (PREFIX && !tile_exists)) {
        loads_only(kbase, vbase, lds_s + (unsigned)((buf ^ 1) * kPKTile));
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) q_load(kb, qnext);
      } else if (wave_last < tile * kPBN + 32) {
        tile_compute_half(tile, buf, kbase, vbase, std::true_type{}, my_row + shift, qnext);
      } else {
        tile_compute(tile, buf, kbase, vbase, std::true_type{}, std::true_type{}, my_row + shift, qnext);
      }
      if (PREFIX) tile_exists = next_exists;
    }
    // Every wave is done with the last tile: its buffer pair is free for the epilogue.  Only LDS traffic is waited for:
    // the loads in flight are the next item's (into the other buffer pair and into qb), which the epilogue does not touch.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // ---- epilogue.  A lane holds 8-byte pieces of its own column, which would make every store instruction touch 64
    //      cache lines; the wave's 32 columns x 256 bytes go through LDS instead (the wave's quarter of the last tile's
    //      buffer pair) and leave as whole 256-byte rows, four per store instruction.  Column n's 16-byte piece P sits at
    //      position P ^ (n & 15) and its two halves are exchanged for the second head's columns: the 32 lanes of a write
    //      pass and the 16 lanes of a read pass then each cover all banks.
    l_run = half_swap_sum(l_run);
    {
      const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
      unsigned char* const stage = lds + (wave < 2 ? buf * kPKTile : 2 * kPKTile + buf * kPTile) + (wave & 1) * 8192;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          u32x2 w;
          w[0] = pack_bf16x2(acc[dt][4 * rq] * inv, acc[dt][4 * rq + 1] * inv);
          w[1] = pack_bf16x2(acc[dt][4 * rq + 2] * inv, acc[dt][4 * rq + 3] * inv);
          *reinterpret_cast<u32x2*>(stage + n * kPRow + (((4 * dt + rq) ^ rloc) << 4) + ((jj ^ hsel) << 3)) = w;
        }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, read back by other lanes
      int piece = lane & 15, c4 = lane >> 4;
      // opaque to the compiler on purpose: otherwise it works the addresses of the eight reads and stores out once, before
      // the item loop, and keeps them in registers it does not have (they were spilled, and reloading them here made every
      // item wait for its own output stores)
      asm volatile("" : "+v"(piece), "+v"(c4));
      uint16_t* const obase = p.out + (int64_t)(cur.seq_begin + wave_row0) * p.o_ts + (int64_t)(2 * cur.unit) * kPD + 8 * piece;
      // all eight reads first, then the eight stores: written as read-store pairs, each store waited for its own read
      u32x4 ow[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int col = 4 * i + c4;           // column of the wave: head i >> 2, row col & 15
        ow[i] = *reinterpret_cast<const u32x4*>(stage + col * kPRow + ((piece ^ (col & 15)) << 4));
        if (i >= 4) ow[i] = u32x4{ow[i][2], ow[i][3], ow[i][0], ow[i][1]};
      }
      __builtin_amdgcn_sched_barrier(0);
      auto out_piece = [&](int i, auto all_rows) {
        const int row = (4 * i + c4) & 15;
        // written once and not read again here: a streaming store leaves less for the write-back at the end of the kernel
        if (decltype(all_rows)::value || wave_row0 + row >= 0)
          __builtin_nontemporal_store(ow[i], reinterpret_cast<u32x4*>(obase + (int64_t)row * p.o_ts + (i >> 2) * kPD));
      };
      stores8 = __builtin_amdgcn_readfirstlane(wave_row0) >= 0;   // rows below 0 only exist in a sequence's first q tile
      if (stores8) {
#pragma unroll
        for (int i = 0; i < 8; ++i) out_piece(i, std::true_type{});
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out_piece(i, std::false_type{});
      }
    }
    buf ^= 1;
    cur = nxt;
    draw = true;
  }

  // ---- the last workgroup to finish clears the counters for the next launch that uses this row
  if (tid == 0) {
    const unsigned done = atomicAdd(&tickets[8], 1u);
    if (done == gridDim.x - 1) {
      for (int c = 0; c < 9; ++c) __hip_atomic_store(&tickets[c], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

int launch_prefill_pair(const PrefillParams& p_in, hipStream_t stream) {
  PrefillParams p = p_in;
  const bool paged = p.block_table != nullptr;
  const bool prefix = paged || p.cu_seqlens_k != p.cu_seqlens || p.total_k_tokens != p.total_tokens;
  if (p.group < 2 || (p.group & 1) || p.batch > kPairMaxBatch) return MOPS_HIP_EUNSUPPORTED;
  PairLaunch L;
  L.table_w = 0;
  L.tiles_per_block = 1;
  if (prefix) {
    // the keys' offsets and the block table are held in LDS; launches too large for that take the other kernel
    if (p.batch > kPairPrefixBatch || (!paged && p.total_k_tokens < 1)) return MOPS_HIP_EUNSUPPORTED;
    // Behind a prefix every item is long, so what this form saves per item and on the diagonal is little; what remains is
    // its finer q tiles (64 rows instead of 128), which pay when sequences bring few new tokens.  With long runs of new
    // tokens the other kernel is the faster one in a sustained series of launches (16 x (1024 + 1024): by 2 %).
    if ((int64_t)p.total_tokens > 512 * (int64_t)p.batch) return MOPS_HIP_EUNSUPPORTED;
    if (paged) {
      if ((int64_t)p.batch * p.max_blocks_per_seq > kPairBlockEntries || p.block_size % kPBN != 0) return MOPS_HIP_EUNSUPPORTED;
      L.table_w = p.max_blocks_per_seq;
      L.tiles_per_block = p.block_size / kPBN;
      p.k_ts = p.v_ts = (int64_t)p.hkv * kPD;   // rows of a cache block
    }
  }
  // m_tiles counts 128-row tiles of the longest sequence; twice as many 64-row tiles bound it here
  L.q_tiles = 2 * p.m_tiles;
  if (L.q_tiles > kPairMaxTiles) return MOPS_HIP_EUNSUPPORTED;
  const int units = p.hq / 2;
  L.classes = p.hkv == 8 ? 8 : 1;
  L.units_per_class = units / L.classes;
  L.units_per_kv = p.group / 2;
  L.upc_shift = -1;
  for (int sft = 0; sft < 16; ++sft)
    if (L.units_per_class == (1 << sft)) L.upc_shift = sft;
  static std::atomic<int> cu_count[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return MOPS_HIP_EUNSUPPORTED;
  int cus = cu_count[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return MOPS_HIP_EUNSUPPORTED;
    cu_count[dev].store(cus, std::memory_order_relaxed);
  }
  // two resident workgroups per CU; fewer when the launch cannot hold that many items
  const int64_t items_bound = ((int64_t)p.total_tokens / kPairRows + p.batch) * L.units_per_class;
  L.members = (int)std::min<int64_t>(items_bound, std::max(1, 2 * cus / L.classes));
  static std::atomic<unsigned> next_slot{0};
  L.slot = (int)(next_slot.fetch_add(1, std::memory_order_relaxed) % kPairSlots);
  const dim3 grid((unsigned)(L.members * L.classes));
  if (prefix) hipLaunchKernelGGL(varlen_prefill_pair_kernel<true>, grid, dim3(kPThreads), 0, stream, p, L);
  else hipLaunchKernelGGL(varlen_prefill_pair_kernel<false>, grid, dim3(kPThreads), 0, stream, p, L);
  return finish_launch();
}

}  // namespace mops
