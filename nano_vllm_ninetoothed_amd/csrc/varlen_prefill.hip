// Varlen (packed THD) causal prefill attention for gfx950, grouped-query heads, head_dim 128.
// bf16 MFMA for both products, fp32 online softmax, K/V tiles staged through LDS.
//
// Work decomposition
//   workgroup (256 lanes, 4 waves) = one 128-row Q tile of one sequence for one query head; wave w owns
//   rows 32w..32w+31; two workgroups per CU.  Tiles with the longest causal prefix are dispatched first,
//   and with 8 kv heads the workgroup id is decoded so that id % 8 — the XCD a workgroup lands on — is
//   the kv head: each XCD's L2 then only ever holds one kv head's K/V.  Ragged batches launch workgroups
//   for existing q tiles only (the kernel maps the workgroup's rank to its tile and sequence).  The output
//   slab of a wave leaves through LDS as whole 256-byte rows.
//
// Per 64-token K/V tile (double-buffered in LDS, one workgroup barrier per tile), hand scheduled: every
// MFMA opens a slot, and what the wave issues while that MFMA runs is fixed by scheduling fences
//   block A   S^T = K . Q^T           16 x v_mfma_f32_32x32x16_bf16 per wave; Q^T stays in registers as
//                                      the B operand; the K operand reads run four MFMAs ahead of use;
//                                      the eight direct-to-LDS loads of the next tile ride in the slots,
//                                      addressed from scalar registers (tile base, LDS destination)
//   block B   softmax head             each lane owns one q row, so the row max is register-local
//                                      (four v_max3 chains) plus one half-wave swap
//                                      (v_permlane32_swap); the score MFMAs start from minus the row's
//                                      reference, which moves lazily; the causal mask is applied only
//                                      on tiles that reach past the wave's first row
//   block C   O^T += V^T . P^T         16 x v_mfma_f32_32x32x16_bf16; the accumulator layout of S^T is
//                                      already the B-operand layout, V^T comes out of LDS through
//                                      ds_read_b64_tr_b16 four MFMAs ahead; the exponent pipeline
//                                      (scale, exp2, sum and pack), skewed one slot per stage, rides in
//                                      the slots (no scale instruction in the form that scales Q once)
// In the steady part of the tile loop the per-tile bookkeeping is two scalar additions.
//
// What was measured on this part and shaped the kernel:
//   * A wave issues a VALU instruction every ~5 cycles (a dependent one every ~9, an exp2 every ~8);
//     two waves of a SIMD together get ~2.8 cycles per instruction.  MFMA and VALU work of the same or
//     of another wave overlap only in part, and a second wave per SIMD adds only ~26 % throughput to
//     this kernel: what counts is the length of a wave's own instruction stream per tile.
//   * Address and bounds bookkeeping between the barrier and the first MFMA took ~900 cycles per tile
//     (a quarter of the tile) before the steady loop replaced it by pointer increments.
//   * Issued in one burst after the barrier, the eight 1-KiB global loads of a wave took ~200 cycles
//     each to issue (all eight waves of the CU queue on the same address path); spread over the MFMA
//     slots the cost vanishes behind the matrix pipe.  Forming a load's address and M0 with vector
//     instructions cost 8 % of the run time; both come from scalar registers now.
//   * Every VALU read of an MFMA result goes through compiler-visible code: the wait states between an
//     MFMA and the first read of its result are software-inserted, and an inline-assembly v_max3 on the
//     scores read half-written registers now and then (results then differ by an ulp from run to run).
//   * Variants that were slower on the benchmark shape: phase-shifting the two waves of a SIMD in
//     256-row, 8-wave workgroups (one in its matrix phase while the other does its softmax; +4 % on
//     8192-token sequences, -10 % on 128..2048-token ones), one wave per SIMD owning two 32-row slabs
//     (512 registers; the compiler shuttles values between the two register files), software-pipelining
//     the two products across half tiles inside a wave (register pressure, two barriers per tile).
//   * Per workgroup there is a fixed cost of ~6.7 us next to ~1.7 - 2.1 us per tile: rank -> tile mapping
//     (1.1 us), issuing the Q and first-tile loads (1.6 us: ~240 cycles per load instruction while the
//     CU's other workgroup streams its tiles), their landing (1 us), the epilogue (1.1 us).  It is the
//     issue of vector-memory instructions, not the latency of the data: pulling the successor's Q into
//     L2 ahead of time made it longer.  A persistent launch (resident workgroups drawing items by
//     ticket) did not shrink it and lengthened the tail; it was 6 % slower on 128..2048-token sequences.
//   * With four waves per CU the transposing read ds_read_b64_tr_b16 delivers ~97 B/clk per CU, a plain
//     ds_read_b64 ~120, ds_read_b128 ~167; each wave reads the whole 16 KiB V tile, and block C's
//     ~1000 cycles track those reads.  With 32 query rows per wave an MFMA consumes 1 KiB of LDS operand
//     per 32 cycles: LDS read bandwidth and matrix rate saturate together.
//   * The shader clock falls to ~1.5 GHz under this kernel on 8192-token sequences (s_memtime against
//     the 100 MHz wall clock; 2.4 GHz idle): counted in cycles the matrix pipe is 72 % busy there.
//
// K/V tiles travel HBM -> LDS directly (global_load_lds_dwordx4, no stop in registers), so LDS rows are unpadded
// (256 B, the two double-buffered tile pairs fill exactly 64 KiB) and bank conflicts are avoided by a swizzle applied
// on the global side of the load: 16-byte position pos of K row r holds piece pos ^ (r & 15), of V row r piece
// pos ^ 4 * (r & 3).  The K operand read (16 consecutive rows, one piece) and the transposing V read (4 rows x 2 x 32
// bytes) then each cover all 64 banks once.  Against staging through registers this removes eight LDS stores and 32
// live registers per tile from every wave's instruction stream (-2 % run time on both benchmark shapes).
#include "prefill_common.h"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace mops {

// PRESCALE: Q is multiplied by softmax_scale * log2(e) when it is read and rounded back to bf16, so the scores leave the
// MFMA as exponents (one VALU instruction per score less).  The rounding costs accuracy in proportion to the size of the
// scores (an error of 2^-9 of a score in the exponent); without it the scale is applied in fp32, as the reference does.
template <bool PRESCALE>
__global__ __launch_bounds__(kPThreads, 2) void varlen_prefill_kernel(const PrefillParams p) {
  // the factor between a score as the MFMA delivers it and the base-2 exponent (the sign of a negative scale is moved into Q)
  // (never exactly zero: a masked score is -inf, and -inf * 0 would be NaN where the probability has to be 0)
  const float ec = PRESCALE ? 1.0f : fmaxf(fabsf(p.scale_log2), 1e-30f);
  // One array, so that the tile buffers start at the workgroup's LDS offset 0 whatever order the compiler lays shared
  // variables out in: a direct-to-LDS load takes its destination from M0 as a plain offset, and every tile offset here
  // stays below 64 KiB.  K[2] then V[2], then per wave the histogram of sequences by q tile count (compact launch).
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kPKTile + 2 * kPTile + (kPThreads / 64) * 68 * 4];
  int (*const lds_hist)[68] = reinterpret_cast<int (*)[68]>(lds + 2 * kPKTile + 2 * kPTile);
  unsigned char* const lds_k = lds;
  unsigned char* const lds_v = lds + 2 * kPKTile;

  // ---- workgroup id -> (q tile m, sequence b, query head h)
  const int idx = blockIdx.x;
  int h, rest;
  if (p.hkv == 8) {  // id % 8 is the XCD: make it the kv head
    const int g8 = idx & 7;
    const int r = (idx >> 3) % p.group;
    rest = (idx >> 3) / p.group;
    h = g8 * p.group + r;
  } else {
    h = idx % p.hq;
    rest = idx / p.hq;
  }
  int b, m;
  int seq_begin, seq_end, kbegin, kend;   // cu_seqlens_q[b], [b+1], cu_seqlens_k[b], [b+1]
  if (p.compact) {
    // `rest` is the rank of this workgroup's (q tile, sequence) pair in the order "highest q tile first,
    // then sequence", counting only pairs that exist: the launch holds no workgroups for tiles past a
    // sequence's end, so the dispatcher never idles on them.  Every wave derives the pair on its own
    // from the tile counts of the sequences (lane l holds sequences l, l + 64, ..).
    // One vector load per array brings every sequence's offsets into the lanes, so the chosen
    // sequence's offsets come out of registers afterwards and not from a second trip to memory.
    const int ln = threadIdx.x & 63;
    int cnt[kPCompactChunks], qs[kPCompactChunks], qe[kPCompactChunks], ks[kPCompactChunks], ke[kPCompactChunks];
#pragma unroll
    for (int j = 0; j < kPCompactChunks; ++j) {
      const int bb = ln + 64 * j;
      qs[j] = qe[j] = ks[j] = ke[j] = 0;
      if (bb < p.batch) {
        qs[j] = p.cu_seqlens[bb];
        qe[j] = p.cu_seqlens[bb + 1];
        ks[j] = p.cu_seqlens_k[bb];
        ke[j] = p.cu_seqlens_k[bb + 1];
      }
    }
#pragma unroll
    for (int j = 0; j < kPCompactChunks; ++j) {
      const int len = min(qe[j], p.total_tokens) - qs[j];
      cnt[j] = (qs[j] >= 0 && len > 0) ? min((len + kPBM - 1) / kPBM, p.m_tiles) : 0;
    }
    int r;   // rank of the pair among the sequences that have tile m
    if (p.m_tiles <= 64) {
      // Lane l works out how many pairs have a q tile index >= l: a histogram of the sequences by tile
      // count (this wave's own, in LDS), its prefix sum N(l) = sequences that have tile l, and the prefix
      // sum of N.  The pair count is non-increasing in l, so one ballot finds the tile index.
      int* const hist = lds_hist[threadIdx.x >> 6];
      hist[ln] = 0;
      if (ln < 4) hist[64 + ln] = 0;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int j = 0; j < kPCompactChunks; ++j)
        if (ln + 64 * j < p.batch) atomicAdd(&hist[cnt[j]], 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const int have = p.batch - wave_prefix_sum(hist[ln]);   // sequences with more than ln tiles
      const int upto = wave_prefix_sum(have);
      const int from = __builtin_amdgcn_readlane(upto, 63) - upto + have;   // pairs with q tile index >= ln
      const unsigned long long reach = __ballot(from > rest);
      if (reach == 0) return;
      m = 63 - __builtin_clzll(reach);
      r = rest - (m < 63 ? __builtin_amdgcn_readlane(from, m + 1) : 0);
    } else {
    // wave-wide sum of small non-negative integers, one ballot per bit (no trip through LDS)
    const int sum_bits = 32 - __builtin_clz((unsigned)(kPCompactChunks * p.m_tiles));
    auto pairs_from = [&](int mm) {   // pairs whose q tile index is >= mm
      int c = 0;
#pragma unroll
      for (int j = 0; j < kPCompactChunks; ++j) c += max(0, cnt[j] - mm);
      int total = 0;
      for (int bit = 0; bit < sum_bits; ++bit) total += __popcll(__ballot((c >> bit) & 1)) << bit;
      return total;
    };
    if (rest >= pairs_from(0)) return;
    int lo = 0, hi = p.m_tiles - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (pairs_from(mid) > rest) lo = mid; else hi = mid - 1;
    }
    m = lo;
    r = rest - pairs_from(m + 1);
    }
    b = -1;
    seq_begin = seq_end = kbegin = kend = 0;
#pragma unroll
    for (int j = 0; j < kPCompactChunks; ++j) {
      const bool has = cnt[j] > m;
      const unsigned long long mask = __ballot(has);
      const int c = __popcll(mask);
      if (b < 0) {
        if (r < c) {
          const int before = __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
          const unsigned long long hit = __ballot(has && before == r);
          const int src = __builtin_ctzll(hit);
          b = 64 * j + src;
          seq_begin = __builtin_amdgcn_readlane(qs[j], src);
          seq_end = __builtin_amdgcn_readlane(qe[j], src);
          kbegin = __builtin_amdgcn_readlane(ks[j], src);
          kend = __builtin_amdgcn_readlane(ke[j], src);
        } else {
          r -= c;
        }
      }
    }
    if (b < 0) return;
  } else {
    b = rest % p.batch;
    m = p.m_tiles - 1 - rest / p.batch;
    seq_begin = p.cu_seqlens[b];
    seq_end = p.cu_seqlens[b + 1];
    if (p.cu_seqlens_k == p.cu_seqlens) {
      kbegin = seq_begin;
      kend = seq_end;
    } else {
      kbegin = p.cu_seqlens_k[b];
      kend = p.cu_seqlens_k[b + 1];
    }
  }
  const int seq_len = min(seq_end, p.total_tokens) - seq_begin;   // query rows of this sequence
  // q tiles are aligned to the END of the sequence: tile m covers rows [q0, q0 + 128) with q0 = len - 128 * (tiles - m),
  // so the partial tile is the first one (q0 < 0, rows below 0 do not exist), which looks at one or two K/V tiles, and
  // not the last one, which looks at all of them: the rows a partial tile leaves idle cost almost nothing there.
  const int seq_tiles = (seq_len + kPBM - 1) / kPBM;
  if (seq_begin < 0 || seq_len <= 0 || m >= seq_tiles) return;
  const int q0 = seq_len - (seq_tiles - m) * kPBM;
  // keys of this sequence: kv_len >= seq_len when a cached prefix precedes the new tokens; query row i
  // then sees keys 0 .. i + shift (bottom-right aligned causal mask)
  int kv_len = kend - kbegin;
  const bool paged = p.block_table != nullptr;
  kv_len = max(0, min(kv_len, paged ? p.max_blocks_per_seq * p.block_size : p.total_k_tokens - kbegin));
  const int shift = kv_len - seq_len;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int n = lane & 31;   // q row inside the wave's 32-row slab (MFMA column)
  const int jj = lane >> 5;  // half: k slice / row-quad selector
  const int g = h / p.group;

  const int kv_end = max(0, min(kv_len, q0 + kPBM + shift));
  const int ntiles = (kv_end + kPBN - 1) / kPBN;
  const int wave_row0 = q0 + 32 * wave;          // first q row (sequence-relative) of this wave
  const int my_row = wave_row0 + n;
  // tiles this wave has to look at: those holding a key visible to one of its rows
  const int my_tiles = max(0, min(ntiles, (wave_row0 + 31 + shift >= 0) ? (wave_row0 + 31 + shift) / kPBN + 1 : 0));

  // ---- cooperative tile loads, HBM -> LDS without a stop in registers (global_load_lds_dwordx4: the 64 lanes of a
  //      wave deposit 64 x 16 bytes at consecutive LDS addresses).  Instruction i of wave w brings rows 16i + 4w .. + 3
  //      of the tile: lane (rr = lane >> 4, pos = lane & 15) fills 16-byte position `pos` of row 16i + 4w + rr.  LDS rows
  //      are unpadded, so bank conflicts are avoided by what a position holds: position pos of row r holds piece
  //      pos ^ (r & 15) of a K row (the operand read of 16 consecutive rows at one piece then covers all banks) and piece
  //      pos ^ 4 * (r & 3) of a V row (the transposing read of 4 rows x 2 x 32 bytes covers all banks).  Rows past the
  //      end of the sequence read the sequence's last row (finite data; their scores are masked, their probabilities
  //      zero); a tile whose cache block does not exist is filled with zeros instead.
  const int ld_row = tid >> 4;     // 4 * wave + rr
  const int ld_pos = tid & 15;
  const int64_t tok_elems = (int64_t)p.hkv * kPD;   // elements between tokens inside a cache block
  const int kcol = g * kPD + ((ld_pos ^ ld_row) << 3);
  const int vcol = g * kPD + ((ld_pos ^ ((ld_row & 3) << 2)) << 3);
  const int32_t* table = paged ? p.block_table + (int64_t)b * p.block_table_row_stride : nullptr;
  auto tile_base = [&](const uint16_t* packed, int64_t ts, int tile, const char*& base, bool& tile_ok) -> bool {
    tile_ok = true;
    if (paged) {
      const int t0 = tile * kPBN;
      const int blk = table[t0 / p.block_size];
      tile_ok = blk >= 0 && blk < p.num_blocks;
      base = reinterpret_cast<const char*>(packed + ((int64_t)(tile_ok ? blk : 0) * p.block_size + (t0 % p.block_size)) * tok_elems);
    } else {
      base = reinterpret_cast<const char*>(packed + (int64_t)(kbegin + tile * kPBN) * ts);
    }
    return tile_ok && (tile + 1) * kPBN <= kv_len;
  };
  // this thread's byte offset of its first piece from a tile's base; piece i lies 16 rows further
  const unsigned k_row_bytes = (unsigned)((paged ? tok_elems : p.k_ts) * 2), v_row_bytes = (unsigned)((paged ? tok_elems : p.v_ts) * 2);
  const unsigned mv_koff0 = (unsigned)ld_row * k_row_bytes + (unsigned)(kcol * 2);
  const unsigned mv_voff0 = (unsigned)ld_row * v_row_bytes + (unsigned)(vcol * 2);
  auto mv_koff = [&](int i) -> unsigned { return mv_koff0 + (unsigned)(16 * i) * k_row_bytes; };
  auto mv_voff = [&](int i) -> unsigned { return mv_voff0 + (unsigned)(16 * i) * v_row_bytes; };
  // Issued as inline assembly on purpose: through the compiler's builtin every later LDS read waits for the load to
  // land (the compiler cannot tell that the buffer being filled is not the buffer being read), which would serialise
  // the tile.  Nothing here depends on the load until the barrier at the top of the next tile, which waits for it
  // explicitly.  M0 carries the wave's LDS destination; lane l deposits its 16 bytes at M0 + 16 * l.
  typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;
  // M0 (the wave's LDS destination) is derived from a vector register inside the statement: a readfirstlane the
  // compiler can see makes it treat the wave index as uniform and restructure the whole tile loop around scalar copies of
  // everything derived from it, at the price of ~70 vector registers.  The statement opens with a wait state because
  // on this chip a v_readfirstlane that directly follows the VALU instruction writing its source register reads the old
  // value; the compiler spaces its own instructions accordingly but does not look inside an asm statement, and the
  // instruction it places right before this one is usually the addition that forms the M0 value.
  const unsigned lds_wave_base = (unsigned)(uintptr_t)(lds_ptr_t)lds + ((unsigned)(tid >> 6) << 10);
  auto to_lds = [&](const char* base, unsigned voff, unsigned lds_off) {   // lds_off: offset of the chunk's tile and row group (wave-uniform value)
    const char* src = base + voff;
    unsigned m0_tmp;
    asm volatile("s_nop 1\n\tv_readfirstlane_b32 %0, %2\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 : "=&s"(m0_tmp) : "v"(src), "v"(lds_wave_base + lds_off) : "memory", "m0");
  };
  // Steady-loop form: the tile's base address and the wave's LDS destination are scalar values (no vector instruction
  // forms an address or M0), the lane's offset from the tile base is one of eight precomputed registers.
  // Both scalar operands are products of scalar arithmetic at every call site (to_scalar() below pays the wait states a
  // VALU-written scalar register needs before a memory instruction may read it); five wait states here instead of one
  // would make the statement safe for any operand and cost 1 % of the run time.
  auto to_lds_s = [&](uint64_t sbase, unsigned voff, unsigned lds_s) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 : : "v"(voff), "s"(sbase), "s"(lds_s) : "memory", "m0");
  };
  // a wave-uniform value the compiler holds in a vector register, moved to a scalar one.  Wait states on both sides,
  // because the compiler's hazard bookkeeping does not see inside the statement: a v_readfirstlane right behind the
  // VALU instruction that writes its source reads the old value, and a memory instruction may not take a scalar
  // register as its base within five cycles of a VALU write to it.
  auto to_scalar = [&](unsigned v) -> unsigned {
    unsigned s_;
    asm volatile("s_nop 1\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(s_) : "v"(v));
    return s_;
  };
  auto to_scalar64 = [&](const void* ptr) -> uint64_t {
    const uint64_t a = reinterpret_cast<uint64_t>(ptr);
    return ((uint64_t)to_scalar((unsigned)(a >> 32)) << 32) | to_scalar((unsigned)a);
  };
  unsigned koff_r[4], voff_r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { koff_r[i] = mv_koff(i); voff_r[i] = mv_voff(i); }
  // offset of instruction i's 1-KiB chunk from the wave's first chunk of tile buffer 0; tile_off: offset of the tile buffer
  auto chunk = [&](unsigned tile_off, int i) -> unsigned { return tile_off + (unsigned)(4 * i) * kPKChunk; };
  // general form (any tile): returns false when the tile's cache block does not exist
  auto load_tile = [&](const uint16_t* packed, int64_t ts, bool is_k, int tile, unsigned tile_off) -> bool {
    const char* base;
    bool tile_ok;
    const bool whole = tile_base(packed, ts, tile, base, tile_ok);
    const unsigned row_bytes = is_k ? k_row_bytes : v_row_bytes;
    const unsigned colb = (unsigned)((is_k ? kcol : vcol) * 2);
    if (!tile_ok) {
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(lds + tile_off + (16 * i + ld_row) * kPRow + (ld_pos << 4)) = u32x4{0u, 0u, 0u, 0u};
    } else if (whole) {
#pragma unroll
      for (int i = 0; i < 4; ++i) to_lds(base, is_k ? mv_koff(i) : mv_voff(i), chunk(tile_off, i));
    } else {
      const int last = kv_len - 1 - tile * kPBN;
#pragma unroll
      for (int i = 0; i < 4; ++i) to_lds(base, (unsigned)min(ld_row + 16 * i, last) * row_bytes + colb, chunk(tile_off, i));
    }
    return tile_ok;
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

  // ---- Q^T as B operand: lane (n, jj) holds Q[my_row][16*kb + 8*jj .. +8) for kb = 0..7.  A lane's own pieces lie 32
  //      bytes apart, so loading them straight into registers makes every load instruction touch 32 cache lines; the
  //      wave's 32 x 256-byte slab instead comes through LDS as eight whole-line direct loads, laid out like a K tile, into
  //      the wave's own 8 KiB of the tile buffers that tile 0 does not use.  Only this wave reads them, and it has done so
  //      before it reaches the first barrier, behind which the loads of tile 1 are issued.  Rows outside the sequence
  //      take a copy of a valid row: rows are independent and theirs are never stored.
  bf16x8 qb[8];
  {
    const unsigned q_lds = (unsigned)kPKTile + (unsigned)(wave & 1) * 8192u + (unsigned)(wave >> 1) * (unsigned)(2 * kPKTile);
    const int64_t q_row_bytes = p.q_ts * 2;
    const char* qbase = reinterpret_cast<const char*>(p.q + (int64_t)seq_begin * p.q_ts + (int64_t)h * kPD);
    const int rr = lane >> 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int rl = 4 * i + rr;
      const int row = min(max(wave_row0 + rl, 0), seq_len - 1);
      const unsigned piece = (unsigned)(ld_pos ^ (rl & 15));
      const char* src_ = qbase + (int64_t)row * q_row_bytes + piece * 16;
      unsigned m0_tmp;
      asm volatile("s_nop 1\n\tv_readfirstlane_b32 %0, %2\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                   : "=&s"(m0_tmp) : "v"(src_), "v"((unsigned)(uintptr_t)(lds_ptr_t)lds + q_lds + (unsigned)(1024 * i)) : "memory", "m0");
    }
  }
  f32x16 acc[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
  float m_run = -INFINITY;  // softmax reference of row my_row, in scaled (base-2 exponent) units
  // the accumulator every score product starts from: minus the reference, so that the MFMA delivers score - reference
  f32x16 s_init;
#pragma unroll
  for (int r = 0; r < 16; ++r) s_init[r] = 0.f;
  float l_run = 0.f;        // this lane's share of the running sum

  // One tile, hand scheduled.  Every MFMA opens a slot; the instructions that follow it up to the next
  // scheduling fence are what the wave issues while that MFMA runs.
  //   block A: S^T = K . Q^T, the eight direct-to-LDS loads of the next tile ride in its slots
  //   block B: row max, whether the reference has to move, the first ten exponentials
  //   block C: O^T += V^T . P^T, the remaining exponentials, the row sums and the bf16 packing ride in its slots
  // `horizon`: last key (sequence-relative) this lane's row may see; only read on the masked variant.
  auto tile_compute = [&](int tile, uint64_t kbase, uint64_t vbase, unsigned lds_s, auto move, auto masked, int horizon) {
    const int buf = tile & 1;
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
        if (decltype(move)::value && (i & 1)) {
          const int j = i >> 1;
          if (j < 4) to_lds_s(kbase, koff_r[j], lds_next + (unsigned)(4 * kPKChunk * j));
          else to_lds_s(vbase, voff_r[j - 4], lds_next + (unsigned)(2 * kPKTile + 4 * kPKChunk * (j - 4)));
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
    // E (exp2) -> P (row sum, bf16 pack) is skewed by one MFMA slot per stage, so nothing issued in a slot
    // depends on anything else issued in it.
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
    // maximum outgrows it by kLazyLog2: probabilities then reach at most 2^kLazyLog2 (harmless in bf16 and in the fp32
    // sums, and the final division by the row sum is exact for any reference), and what a move costs (64 accumulator
    // multiplies, 32 subtractions on this tile's scores, 16 moves for s_init), behind which nothing else can be issued,
    // runs on a row's first tile or two instead of on every other tile.
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
    float f0[16], f1[16];   // per element pair q = 0..15 (elements 2q, 2q+1 of this lane's 32 scores): stage values
    auto stage_e = [&](int q) {
      const int tt = q >> 3, r = 2 * (q & 7);
      f0[q] = __builtin_amdgcn_exp2f(PRESCALE ? s[tt][r] : s[tt][r] * ec);
      f1[q] = __builtin_amdgcn_exp2f(PRESCALE ? s[tt][r + 1] : s[tt][r + 1] * ec);
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
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    l_run = l_run * alpha + (ps0 + ps1);
  };

  // The same for a tile of which no row of this wave sees more than the first 32 keys (a wave's last tile on the
  // diagonal, every other time): the fully masked half is neither multiplied nor exponentiated.  Eight MFMAs per block.
  auto tile_compute_half = [&](int tile, uint64_t kbase, uint64_t vbase, unsigned lds_s, auto move, int horizon) {
    const int buf = tile & 1;
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
        if (decltype(move)::value) {
          if (i < 4) to_lds_s(kbase, koff_r[i], lds_next + (unsigned)(4 * kPKChunk * i));
          else to_lds_s(vbase, voff_r[i - 4], lds_next + (unsigned)(2 * kPKTile + 4 * kPKChunk * (i - 4)));
        }
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
      f0[q] = __builtin_amdgcn_exp2f(PRESCALE ? s0[2 * q] : s0[2 * q] * ec);
      f1[q] = __builtin_amdgcn_exp2f(PRESCALE ? s0[2 * q + 1] : s0[2 * q + 1] * ec);
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
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    l_run = l_run * alpha + (ps0 + ps1);
  };

  // ---- tile loop.  The next tile travels HBM -> the other LDS buffer during block A; that buffer was last read before
  //      this tile's barrier, and the barrier at the top of the next tile waits for the loads to have landed.
  bool tile_exists = true;
  if (ntiles > 0) {
    tile_exists = load_tile(p.k, p.k_ts, true, 0, 0u);
    load_tile(p.v, p.v_ts, false, 0, 2u * kPKTile);
  }
  {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned char* qt = lds + kPKTile + (wave & 1) * 8192 + (wave >> 1) * (2 * kPKTile);
#pragma unroll
    for (int kb = 0; kb < 8; ++kb) {
      // PRESCALE: Q is scaled by softmax_scale * log2(e) here, once, and rounded back to bf16: the scores then come out
      // of the MFMA in the exponent's units and the softmax spends no instruction on scaling them
      u32x4 w = *reinterpret_cast<const u32x4*>(qt + rd_k[kb]);
      if (PRESCALE) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w[e] = pack_bf16x2(__builtin_bit_cast(float, w[e] << 16) * p.scale_log2, __builtin_bit_cast(float, w[e] & 0xffff0000u) * p.scale_log2);
      } else if (p.scale_log2 < 0.f) {
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] ^= 0x80008000u;   // -Q, exactly
      }
      qb[kb] = __builtin_bit_cast(bf16x8, w);
    }
  }
#pragma unroll
  for (int kb = 0; kb < 8; ++kb) asm volatile("" : "+v"(qb[kb]));
  // Steady prefix of the loop: tiles this wave computes and whose successor is a whole tile.  There the
  // per-tile bookkeeping is two scalar additions; everything else (partial tiles, the last tile, tiles this
  // wave skips, paged sequences of more than 64 blocks or with a missing block) takes the general loop below.  Both loops hold
  // exactly one barrier per tile, so the waves of a workgroup may sit in different ones.
  int tile = 0;
  {
    // Paged caches take the steady loop when the sequence's keys lie in at most 64 cache blocks, all of which exist:
    // lane l holds block l's table entry, a tile's base comes out of it by a lane read (a scalar value, no trip to
    // memory inside the loop), and inside a block the base advances by one tile's bytes.
    int entry = 0;
    bool steady = true;
    int tiles_per_block = 1;
    if (paged) {
      const int used_blocks = (kv_len + p.block_size - 1) / p.block_size;
      if (lane < used_blocks) entry = table[lane];   // used_blocks > 64: not taken below
      const bool entry_ok = lane >= used_blocks || (entry >= 0 && entry < p.num_blocks);
      steady = used_blocks <= 64 && __all(entry_ok);
      tiles_per_block = p.block_size / kPBN;
    }
    const int n_fast = steady ? min(my_tiles, min(kv_len / kPBN - 1, ntiles - 1)) : 0;
    const int unmasked = wave_row0 + shift + 1 >= 0 ? (wave_row0 + shift + 1) / kPBN : 0;   // tiles wholly below the first row's horizon
    // byte distance between consecutive tiles of a packed K / V, or of a cache block
    const uint64_t kstep = (uint64_t)kPBN * (uint64_t)(paged ? tok_elems : p.k_ts) * 2u, vstep = (uint64_t)kPBN * (uint64_t)(paged ? tok_elems : p.v_ts) * 2u;
    const uint64_t block_bytes = (uint64_t)p.block_size * (uint64_t)tok_elems * 2u;
    const unsigned lds_s = to_scalar(lds_wave_base);
    // base of the tile after the one being computed (tile 1 to begin with)
    uint64_t kbase, vbase;
    int blk_i = 1 / tiles_per_block, in_blk = 1 % tiles_per_block;
    if (paged) {
      const uint64_t off = (uint64_t)(unsigned)__builtin_amdgcn_readlane(entry, blk_i & 63) * block_bytes + (uint64_t)in_blk * kstep;
      kbase = reinterpret_cast<uint64_t>(p.k) + off;
      vbase = reinterpret_cast<uint64_t>(p.v) + off;
    } else {
      kbase = to_scalar64(p.k + (int64_t)(kbegin + kPBN) * p.k_ts);
      vbase = to_scalar64(p.v + (int64_t)(kbegin + kPBN) * p.v_ts);
    }
    for (; tile < n_fast; ++tile) {
      tile_barrier();
      if (tile < unmasked) tile_compute(tile, kbase, vbase, lds_s, std::true_type{}, std::false_type{}, 0);
      else if (wave_row0 + 31 + shift < tile * kPBN + 32) tile_compute_half(tile, kbase, vbase, lds_s, std::true_type{}, my_row + shift);
      else tile_compute(tile, kbase, vbase, lds_s, std::true_type{}, std::true_type{}, my_row + shift);
      if (paged && ++in_blk == tiles_per_block) {
        in_blk = 0;
        ++blk_i;
        const uint64_t off = (uint64_t)(unsigned)__builtin_amdgcn_readlane(entry, blk_i & 63) * block_bytes;
        kbase = reinterpret_cast<uint64_t>(p.k) + off;
        vbase = reinterpret_cast<uint64_t>(p.v) + off;
      } else {
        kbase += kstep;
        vbase += vstep;
      }
    }
  }
  for (; tile < ntiles; ++tile) {
    tile_barrier();
    bool next_exists = true;
    if (tile + 1 < ntiles) {
      next_exists = load_tile(p.k, p.k_ts, true, tile + 1, (unsigned)((tile + 1) & 1) * kPKTile);
      load_tile(p.v, p.v_ts, false, tile + 1, 2u * kPKTile + (unsigned)((tile + 1) & 1) * kPTile);
    }
    // the mask is only needed where the tile holds a key beyond the first row's horizon; a tile whose cache
    // block does not exist (it was filled with zeros) is masked as a whole: its keys get no weight, as in decode
    const bool masked = tile * kPBN + kPBN - 1 > wave_row0 + shift || !tile_exists;
    const int horizon = tile_exists ? my_row + shift : -1;
    if (tile < my_tiles) {
      if (tile_exists && wave_row0 + 31 + shift < tile * kPBN + 32) tile_compute_half(tile, 0, 0, 0u, std::false_type{}, horizon);
      else if (masked) tile_compute(tile, 0, 0, 0u, std::false_type{}, std::true_type{}, horizon);
      else tile_compute(tile, 0, 0, 0u, std::false_type{}, std::false_type{}, 0);
    }
    tile_exists = next_exists;
  }
  tile_barrier();   // every wave is done with the last tile: the whole of LDS is free for the epilogue

  // ---- epilogue.  A lane holds 8-byte pieces of its own row, which would make every store instruction
  //      touch 64 cache lines; the wave's 32 x 128 slab goes through LDS instead and leaves as whole
  //      256-byte rows, four per store instruction.  The staging area is the start of the tile buffers:
  //      no wave reads a tile any more once all have passed the barrier above.
  l_run = half_swap_sum(l_run);
  {
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    constexpr int kOStride = 272;   // bytes between staged rows (padded: the 8-byte pieces of 32 rows spread over the banks)
    unsigned char* const stage = lds + wave * 32 * kOStride;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        u32x2 w;
        w[0] = pack_bf16x2(acc[dt][4 * rq] * inv, acc[dt][4 * rq + 1] * inv);
        w[1] = pack_bf16x2(acc[dt][4 * rq + 2] * inv, acc[dt][4 * rq + 3] * inv);
        *reinterpret_cast<u32x2*>(stage + n * kOStride + 64 * dt + 16 * rq + 8 * jj) = w;
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, read back by other lanes
    int piece = lane & 15, row4 = lane >> 4;
    // opaque to the compiler on purpose: otherwise it recognises the row numbers of the Q loads at the top of the kernel
    // and keeps eight registers of them alive through the tile loop
    asm volatile("" : "+v"(piece), "+v"(row4));
    uint16_t* const obase = p.out + (int64_t)(seq_begin + wave_row0) * p.o_ts + (int64_t)h * kPD + 8 * piece;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = row4 + 4 * i;
      const u32x4 w = *reinterpret_cast<const u32x4*>(stage + row * kOStride + 16 * piece);
      // written once and not read again here: a streaming store leaves less for the write-back at the end of the kernel
      if (wave_row0 + row >= 0 && wave_row0 + row < seq_len) __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(obase + (int64_t)row * p.o_ts));
    }
  }
}

// MOPS_HIP_PREFILL_PRESCALE=1 selects the form that scales Q once (read at the first call)
static bool prefill_prescale() {
  static const bool on = [] {
    const char* e = getenv("MOPS_HIP_PREFILL_PRESCALE");
    return e && e[0] == '1';
  }();
  return on;
}

static bool prefill_force_rows() {
  static const bool on = [] {
    const char* e = getenv("MOPS_HIP_PREFILL_FORM");
    return e && e[0] == 'r';
  }();
  return on;
}

}  // namespace mops

extern "C" int mops_hip_attn_varlen_causal_bf16(const void* q, int64_t q_token_stride,
                                                const void* k, int64_t k_token_stride,
                                                const void* v, int64_t v_token_stride,
                                                void* out, int64_t out_token_stride,
                                                const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                                const int32_t* block_table, int64_t block_table_row_stride,
                                                int64_t block_size, int64_t num_blocks, int64_t max_blocks_per_seq,
                                                int64_t batch, int64_t total_tokens, int64_t total_k_tokens,
                                                int64_t max_seqlen_q,
                                                int64_t hq, int64_t hkv, int64_t head_dim,
                                                float softmax_scale,
                                                void* stream) {
  using namespace mops;
  if (batch < 0 || total_tokens < 0 || total_k_tokens < 0 || max_seqlen_q < 0 || hq <= 0 || hkv <= 0) return MOPS_HIP_EINVAL;
  if (batch == 0 || total_tokens == 0 || max_seqlen_q == 0) return MOPS_HIP_OK;
  if (!q || !k || !v || !out || !cu_seqlens_q) return MOPS_HIP_EINVAL;
  if (hq % hkv != 0) return MOPS_HIP_EINVAL;
  if (head_dim != kPD) return MOPS_HIP_EUNSUPPORTED;
  if (q_token_stride < hq * kPD || out_token_stride < hq * kPD) return MOPS_HIP_EINVAL;
  if (total_tokens > 0x3fffffffLL || total_k_tokens > 0x3fffffffLL || batch > (1 << 20) || hq > 4096) return MOPS_HIP_EUNSUPPORTED;
  if ((q_token_stride & 7) || (out_token_stride & 7)) return MOPS_HIP_EALIGN;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return MOPS_HIP_EALIGN;
  if (block_table) {
    if (!cu_seqlens_k || block_size <= 0 || num_blocks <= 0 || max_blocks_per_seq <= 0 ||
        block_table_row_stride < max_blocks_per_seq)
      return MOPS_HIP_EINVAL;
    if (block_size % kPBN != 0 || num_blocks * block_size > (int64_t)0x7fffffff || max_blocks_per_seq * block_size > (1 << 24))
      return MOPS_HIP_EUNSUPPORTED;
  } else {
    if (k_token_stride < hkv * kPD || v_token_stride < hkv * kPD) return MOPS_HIP_EINVAL;
    if ((k_token_stride & 7) || (v_token_stride & 7)) return MOPS_HIP_EALIGN;
    // a lane's byte offset inside a 64-token tile is kept in 32 bits
    if (k_token_stride > (1ll << 24) || v_token_stride > (1ll << 24)) return MOPS_HIP_EUNSUPPORTED;
    if (!cu_seqlens_k && total_k_tokens != total_tokens) return MOPS_HIP_EINVAL;
  }
  if (max_seqlen_q > total_tokens) max_seqlen_q = total_tokens;

  PrefillParams p;
  p.q = (const uint16_t*)q;
  p.k = (const uint16_t*)k;
  p.v = (const uint16_t*)v;
  p.out = (uint16_t*)out;
  p.q_ts = q_token_stride;
  p.k_ts = k_token_stride;
  p.v_ts = v_token_stride;
  p.o_ts = out_token_stride;
  p.cu_seqlens = cu_seqlens_q;
  p.cu_seqlens_k = cu_seqlens_k ? cu_seqlens_k : cu_seqlens_q;
  p.block_table = block_table;
  p.block_table_row_stride = block_table_row_stride;
  p.block_size = (int)block_size;
  p.num_blocks = (int)num_blocks;
  p.max_blocks_per_seq = (int)max_blocks_per_seq;
  p.batch = (int)batch;
  p.total_tokens = (int)total_tokens;
  p.total_k_tokens = (int)total_k_tokens;
  p.m_tiles = (int)((max_seqlen_q + kPBM - 1) / kPBM);
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.group = (int)(hq / hkv);
  p.scale_log2 = softmax_scale * 1.44269504088896340736f;
  // Every sequence has ceil(len / 128) q tiles, at most total_tokens / 128 + batch in all.  When that is
  // clearly fewer than the m_tiles x batch rectangle (ragged lengths) and there are at most 256
  // sequences, the kernel maps workgroup ids onto the existing tiles only; the mapping costs each
  // workgroup one more trip to memory, so equal-length batches keep the rectangle.
  int64_t pairs = (int64_t)p.m_tiles * batch;
  const int64_t pairs_bound = total_tokens / kPBM + batch;
  p.compact = batch <= 64 * kPCompactChunks && pairs_bound * 10 < pairs * 9;
  if (p.compact) pairs = pairs_bound;
  const int64_t grid = pairs * hq;
  if (grid > 0x7fffffffLL) return MOPS_HIP_EUNSUPPORTED;
  // Grouped-query heads in pairs take the form that packs two heads into a wave and keeps workgroups resident
  // (varlen_prefill_pair.hip), with or without a cached prefix; everything else (odd group sizes, very large batches, a
  // cached prefix with more than 64 sequences or a block table of more than 768 entries, the form that scales Q once)
  // stays here.  MOPS_HIP_PREFILL_FORM=rows forces this kernel.
  if (!prefill_prescale() && !prefill_force_rows()) {
    const int st = launch_prefill_pair(p, (hipStream_t)stream);
    if (st != MOPS_HIP_EUNSUPPORTED) return st;
  }
  if (prefill_prescale())
    hipLaunchKernelGGL(varlen_prefill_kernel<true>, dim3((unsigned)grid), dim3(kPThreads), 0, (hipStream_t)stream, p);
  else
    hipLaunchKernelGGL(varlen_prefill_kernel<false>, dim3((unsigned)grid), dim3(kPThreads), 0, (hipStream_t)stream, p);
  return finish_launch();
}
