// bfloat16 attention over the paged cache on the matrix cores (16x16x32 MFMA, float32 softmax).
//
// Both kernels walk the keys 32 at a time and keep everything in registers:
//   S^T[key, row]  = K[key, :] . Q[row, :]         A = 16 keys of K (16-byte loads per lane), B = Q
//   O^T[dim, row] += V^T[dim, key] . P^T[key, row]  A = V^T (the value pool is stored [dim][key]), B = P
// The MFMA result layout of S^T (4 consecutive keys per lane for one row) is exactly the B-operand
// layout of P^T once the 32 keys of a step are numbered (group of 4, tile) instead of in order, and
// V^T is loaded with the same numbering, so probabilities never leave registers.
//
// Prefill: one wave per (tile of 16 * NQT queries of one sequence, head); with pages of a power of two,
// the staged kernel below (keys and values through LDS, shared by several heads and split between waves).
// Decode (one query per sequence): one block per (256 keys, key/value head, sequence); the rows of
// the MFMA are the query heads of the group, so keys and values are read once per group.  The four
// waves take 64 keys each and are merged in LDS; blocks are merged by a second small kernel.  (Letting
// the block that finishes last do the merge needs a device-wide fence in every block, whose cache
// write-back cost more than the second launch: measured 2.0 ms against 1.4 ms per step.)
// Keys are always cut at the same places, so a position's result does not depend on the batch.
#include <type_traits>

#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kDecodeChunk = 256;   // keys per decode block
constexpr int kDecodeWaveKeys = 64; // keys per wave of a decode block

struct PagedKV {
  const uint16_t* k;     // key pool, already offset to the key/value head: + page * page_stride + slot * HD + d
  const uint16_t* v;     // value pool, offset to the head: + page * page_stride + d * page_size + slot
  const int32_t* table;  // this sequence's block table, from entry `table_first` on
  int page_size, num_pages;
  size_t page_stride;    // elements between pages: nkv * page_size * HD
  int table_first = 0;   // the table entry that table[0] is (a copy of a part of the table starts later)
  int page_shift = 0;    // POW2: page_size == 1 << page_shift
};

// Which page of the sequence a key lies in, and where in that page.  A division by a number that only the
// launch knows is some forty vector instructions; pages of a power of two of tokens (POW2) need a shift.
template <bool POW2>
__device__ __forceinline__ int page_index(const PagedKV& kv, int key) {
  return POW2 ? key >> kv.page_shift : key / kv.page_size;
}
template <bool POW2>
__device__ __forceinline__ int page_offset(const PagedKV& kv, int key) {
  return POW2 ? key & (kv.page_size - 1) : key % kv.page_size;
}
template <bool POW2>
__device__ __forceinline__ int page_of(const PagedKV& kv, int key) {
  const int page = kv.table[page_index<POW2>(kv, key) - kv.table_first];
  return min(max(page, 0), kv.num_pages - 1);   // a bad table entry must not become a wild address
}

// Keys and values of one step of 32 keys, as MFMA operands in registers.
template <int DT>
struct KVStep {
  bf16x8 ka[2][(DT + 1) / 2];   // K rows: tile of 16 keys x chunks of 32 dims
  uint2 va[DT][2];              // V^T rows: 16 dims x (4 keys of tile 0, 4 keys of tile 1)
};

// Requests the 32 keys starting at key0 (a multiple of 32).  Loads are clamped to keys in [k_lo, k_hi];
// what lies outside is masked by position when the step is used.
template <int DT, bool POW2 = false>
__device__ __forceinline__ void load_step(KVStep<DT>& r, const PagedKV& kv, int key0, int k_lo, int k_hi) {
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2;
  const int lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    const int key = min(max(key0 + 16 * kt + lr, k_lo), k_hi);
    const uint16_t* krow = kv.k + size_t(page_of<POW2>(kv, key)) * kv.page_stride + size_t(page_offset<POW2>(kv, key)) * HD;
#pragma unroll
    for (int c = 0; c < HC; ++c) {
      const int d0 = 32 * c + 8 * lj;
      r.ka[kt][c] = d0 < HD ? as_bf16x8(ldg128(krow + d0)) : as_bf16x8(make_uint4(0, 0, 0, 0));
    }
  }
  // V^T operands: row = dim 16 * dt + lr; k slots (lj, 0..3) = keys key0 + 4 lj + 0..3, (lj, 4..7) = the same + 16
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
    int kb = key0 + 16 * kt + 4 * lj;
    kb = min(max(kb, (k_lo >> 2) << 2), (k_hi >> 2) << 2);
    const uint16_t* vbase = kv.v + size_t(page_of<POW2>(kv, kb)) * kv.page_stride + page_offset<POW2>(kv, kb);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      r.va[dt][kt] = *reinterpret_cast<const uint2*>(vbase + size_t(16 * dt + lr) * kv.page_size);
  }
}

constexpr float kNoKeyYet = -1.0e30f;   // running maximum before any key: finite, so that no inf - inf arises
// The running maximum of a row follows the true maximum only when that has grown by more than this (in
// log2 units): until then the probabilities are taken against the older maximum and are at most 2^8, which
// float32 sums and bfloat16 operands hold as exactly as values below 1, and the accumulators are not rescaled.
constexpr float kRescaleStep = 8.0f;

// max(a, b) as the median of (a, b, +inf): one instruction, where fmaxf of an MFMA result costs a
// canonicalising self-maximum more.  (Not inline assembly: the compiler must see who reads MFMA and
// lane-swap results, to keep the wait states those need.)
__device__ __forceinline__ float vmax(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }
__device__ __forceinline__ float vmax3(float a, float b, float c) { return vmax(vmax(a, b), c); }
// Maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48, in the vector unit (no trip through LDS).
__device__ __forceinline__ float max_over_quarters(float x) {
  const unsigned u = __float_as_uint(x);
  const auto h = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const unsigned v = __float_as_uint(vmax(__uint_as_float(h[0]), __uint_as_float(h[1])));
  const auto f = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return vmax(__uint_as_float(f[0]), __uint_as_float(f[1]));
}

// Scores, running softmax and P.V of one loaded step for NQT tiles of 16 rows.
// qpos[qt]: position of this lane's row (column l % 16 of tile qt), or -1 for a row that does not exist.
// MASKED false: every key of the step is visible to every existing row (the caller has checked), and
// rows that do not exist compute values nobody reads.  The running maximum m is in log2 units and
// starts at kNoKeyYet.
// CONTIG: the step's keys in the order 8 lj + 4 kt + r (a lane's eight keys in a row, as the staged kernel reads its
// values from LDS in one piece) instead of 16 kt + 4 lj + r; whoever loads the step lays its key rows out to match.
template <int DT, int NQT, bool MASKED, bool LAZY, bool CONTIG>
__device__ __forceinline__ void attend_step_impl(const KVStep<DT>& r, const bf16x8 (&qop)[NQT][(DT + 1) / 2],
                                                 floatx4 (&o)[NQT][DT], float (&m)[NQT], float (&lsum)[NQT],
                                                 int key0, int k_lo, const int (&qpos)[NQT], int window,
                                                 float scale2) {
  constexpr int HC = (DT + 1) / 2;
  const int lane = threadIdx.x & 63, lj = lane >> 4;

  floatx4 s[NQT][2];
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      s[qt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < HC; ++c) s[qt][kt] = mfma16(r.ka[kt][c], qop[qt][c], s[qt][kt]);
    }

  float raw[NQT];
  bool grown = false;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (MASKED) {
      // visible keys of this lane's row: lo .. lo + span (none when span < 0), tested with one unsigned compare
      const int hi = qpos[qt];
      const int lo = window > 0 ? max(k_lo, hi - window + 1) : k_lo;
      const int span = hi - lo;
      const unsigned limit = span >= 0 ? unsigned(span) : 0u;
      const int base = span >= 0 ? lo : key0 + 64;          // key - base < 0 for every key of the step: none passes
      const int first = key0 + (CONTIG ? 8 : 4) * lj - base;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
          s[qt][kt][r4] = unsigned(first + (CONTIG ? 4 : 16) * kt + r4) <= limit ? s[qt][kt][r4] : -INFINITY;
    }
    raw[qt] = vmax3(s[qt][0][0], s[qt][0][1], s[qt][0][2]);
    raw[qt] = vmax3(raw[qt], s[qt][0][3], s[qt][1][0]);
    raw[qt] = vmax3(raw[qt], s[qt][1][1], s[qt][1][2]);
    raw[qt] = vmax(raw[qt], s[qt][1][3]);
    // LAZY: the lane's own 8 keys decide whether anything has to be done about the maximum, and the row's other
    // three lanes are asked only then (-inf when the lane sees no key of the step): ten instructions less per
    // step and tile of rows.  Otherwise the row's maximum is formed first.
    if (!LAZY) raw[qt] = max_over_quarters(raw[qt]);
    grown = grown || raw[qt] * scale2 > m[qt] + kRescaleStep;
  }
  // One test for all the tiles of rows: the code that follows it is then one straight run for all of them, which
  // the compiler interleaves (a test a tile cut it into pieces that each waited for its own chain of exponentials
  // and matrix instructions).  A tile whose maximum has not grown goes through the rescaling with a factor of one.
  if (__builtin_amdgcn_ballot_w64(grown) != 0) {
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      const float top = (LAZY ? max_over_quarters(raw[qt]) : raw[qt]) * scale2;
      const float mx = top > m[qt] + kRescaleStep ? top : m[qt];   // finite: m starts finite
      const float alpha = __builtin_amdgcn_exp2f(m[qt] - mx);
      m[qt] = mx;
      lsum[qt] *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[qt][dt] *= alpha;
    }
  }
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const float mx = m[qt];
    float p[2][4], sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        p[kt][r4] = __builtin_amdgcn_exp2f(fmaf(s[qt][kt][r4], scale2, -mx));   // exp2(-inf) = 0 for masked keys
        sum += p[kt][r4];
      }
    lsum[qt] += sum;
    const uint4 pb = make_uint4(pack_bf16x2(p[0][0], p[0][1]), pack_bf16x2(p[0][2], p[0][3]),
                                pack_bf16x2(p[1][0], p[1][1]), pack_bf16x2(p[1][2], p[1][3]));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint4 a = make_uint4(r.va[dt][0].x, r.va[dt][0].y, r.va[dt][1].x, r.va[dt][1].y);
      o[qt][dt] = mfma16(as_bf16x8(a), as_bf16x8(pb), o[qt][dt]);
    }
  }
}

// `first_pos`: smallest position among the rows that exist; a step whose 32 keys all lie at or before
// it (and inside [k_lo, ...) with no window) needs no masking.
template <int DT, int NQT, bool LAZY = true, bool CONTIG = false>
__device__ __forceinline__ void attend_step(const KVStep<DT>& r, const bf16x8 (&qop)[NQT][(DT + 1) / 2],
                                            floatx4 (&o)[NQT][DT], float (&m)[NQT], float (&lsum)[NQT], int key0,
                                            int k_lo, const int (&qpos)[NQT], int window, float scale2,
                                            int first_pos) {
  if (window <= 0 && key0 >= k_lo && key0 + 31 <= first_pos)
    attend_step_impl<DT, NQT, false, LAZY, CONTIG>(r, qop, o, m, lsum, key0, k_lo, qpos, window, scale2);
  else
    attend_step_impl<DT, NQT, true, LAZY, CONTIG>(r, qop, o, m, lsum, key0, k_lo, qpos, window, scale2);
}

template <int DT>
__device__ __forceinline__ void load_q_operand(bf16x8 (&qop)[(DT + 1) / 2], const uint16_t* qrow) {
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2;
  const int lj = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int c = 0; c < HC; ++c) {
    const int d0 = 32 * c + 8 * lj;
    qop[c] = (qrow && d0 < HD) ? as_bf16x8(ldg128(qrow + d0)) : as_bf16x8(make_uint4(0, 0, 0, 0));
  }
}

// ------------------------------------------------------------------------------------------ prefill
template <int DT, int NQT>
__global__ __launch_bounds__(64) void attention_prefill_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pool,
    const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ tiles, uint16_t* __restrict__ out, int nq, int nkv, int page_size, int num_pages,
    int window, float scale2) {
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2;
  const int seq = tiles[2 * blockIdx.x], q_off = tiles[2 * blockIdx.x + 1];
  const int h = blockIdx.y, g = h / (nq / nkv);
  const int qlen = q_len[seq], ctx = ctx_len[seq], qs = q_start[seq];
  const int nvalid = min(16 * NQT, qlen - q_off);
  if (nvalid <= 0) return;
  const int pos0 = ctx - qlen + q_off;
  const int lane = threadIdx.x, lr = lane & 15, lj = lane >> 4;

  PagedKV kv;
  kv.page_size = page_size;
  kv.num_pages = num_pages;
  kv.page_stride = size_t(nkv) * page_size * HD;
  kv.k = k_pool + size_t(g) * page_size * HD;
  kv.v = v_pool + size_t(g) * page_size * HD;
  kv.table = block_tables + size_t(seq) * max_blocks;

  bf16x8 qop[NQT][HC];
  int qpos[NQT];
  floatx4 o[NQT][DT];
  float m[NQT], lsum[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int row = 16 * qt + lr;
    const bool valid = row < nvalid;
    qpos[qt] = valid ? pos0 + row : -1;
    load_q_operand<DT>(qop[qt], valid ? q + size_t(qs + q_off + row) * q_stride + h * HD : nullptr);
    m[qt] = kNoKeyYet;
    lsum[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const int k_hi = pos0 + nvalid - 1;
  const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  // the next step's keys and values are on their way while the current step is multiplied
  KVStep<DT> cur, nxt;
  int key0 = (k_lo >> 5) << 5;
  load_step<DT>(cur, kv, key0, k_lo, k_hi);
  for (; key0 <= k_hi; key0 += 32) {
    const bool more = key0 + 32 <= k_hi;
    if (more) load_step<DT>(nxt, kv, key0 + 32, k_lo, k_hi);
    attend_step<DT, NQT>(cur, qop, o, m, lsum, key0, k_lo, qpos, window, scale2, pos0);
    if (more) cur = nxt;
  }

#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    float l = lsum[qt];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int row = 16 * qt + lr;
    if (row >= nvalid) continue;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* dst = out + size_t(qs + q_off + row) * (size_t(nq) * HD) + h * HD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {   // lane holds dims 16 dt + 4 lj + 0..3 of its row
      const floatx4 v = o[qt][dt] * inv;
      *reinterpret_cast<uint2*>(dst + 16 * dt + 4 * lj) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    }
  }
}

// ------------------------------------------------------------------------------------------ prefill, staged
// One block per (tile of 16 * NQT queries, HPB heads of one key/value head): a team of WPT waves per head.
// The keys are walked in stages of 128 that the block copies into LDS once for all its teams; wave w of
// a team takes its share of every stage (128 / WPT keys, 32 at a time) with a running softmax of its own, and the waves
// are merged in LDS at the end.  Against one wave walking all keys this cuts the chain of dependent steps
// by four; sharing a stage between heads cuts the traffic from L2, which bounds the kernel.
// The sequence's page numbers are copied to LDS first, so that a fetch is one trip to memory.
// Needs pages of 8, 16, 32, ... tokens (a power of two).
constexpr int kStageKeys = 128;
// LDS row of key r of a stage: the keys of each step of 32 lie in the order in which the two score tiles take them
// (attend_step's CONTIG order): key 8 a + 4 t + b of the step in row 16 t + 4 a + b, so that lane row 4 a + b of
// tile t reads row 16 t + (its own number) as it would without the permutation.
__device__ __forceinline__ constexpr int step_row(int r) { return (r & ~31) | ((r & 4) << 2) | (((r & 31) >> 3) << 2) | (r & 3); }
constexpr int kMaxTableLds = 2048;    // page numbers held in LDS; longer tables are read from memory

template <int DT, int NQT, int HPB, int WPT, bool AHEAD, bool PAIRED>
__global__ __launch_bounds__(64 * WPT * HPB) void attention_prefill_staged_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pool,
    const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ tiles, uint16_t* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, int n_splits, int stages_per_split, int nq, int nkv, int page_shift, int num_pages,
    int window, float scale2, int n_tiles) {
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2;
  constexpr int THREADS = 64 * WPT * HPB;
  constexpr int WAVE_KEYS = kStageKeys / WPT;          // keys of a stage that one wave of a team takes
  // Key row pitch in LDS (elements).  A 16-byte LDS read serves lanes {0-3, 12-15, 20-27} of each half-wave in
  // one pass and the other 16 in a second (measured with two lanes at a time on one bank), not 16 lanes in a
  // row: with 16 bytes of padding the rows of those lanes met two to a bank (8 cycles an instruction instead
  // of 4); 32 bytes of padding keep them apart while the row is a whole number of 64 bytes.
  constexpr int KP = HD + (DT % 2 == 0 ? 16 : 8);
  // Value row pitch: the stage's keys + 32 bytes, for the same reason.  A lane reads its eight keys of a step in
  // one piece of 16 bytes (4 cycles an instruction); as two pieces of 8 bytes 32 bytes apart the compiler made one
  // ds_read2_b64 of them, which took 16 cycles at the old pitch and 8 at the best (counted on the pattern alone).
  constexpr int VP = kStageKeys + 16;
  constexpr int KCHUNKS = kStageKeys * (HD / 8);      // 16-byte pieces of the stage's keys ...
  const int page_size = 1 << page_shift, page_mask = page_size - 1;   // pages are a power of two of tokens
  constexpr int CHUNKS = 2 * KCHUNKS;                 // ... and of its values
  constexpr int PER_THREAD = (CHUNKS + THREADS - 1) / THREADS;
  constexpr int STAGE_BYTES = (kStageKeys * KP + HD * VP) * 2;
  constexpr int MERGE_BYTES = WPT * 16 * NQT * (HD + 4) * 4;
  __shared__ __attribute__((aligned(16))) unsigned char smem[STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES];
  __shared__ int32_t s_table[kMaxTableLds];
  uint16_t* ks = reinterpret_cast<uint16_t*>(smem);
  uint16_t* vs = ks + kStageKeys * KP;

  // Tiles are listed in order of position; the last ones walk the most keys, so they start first.  PAIRED: a
  // block takes tile n - 1 - b and then tile b, a long walk and a short one, so that all blocks walk about as
  // many keys.  (When all blocks of a causal prompt fit on the chip at once, nothing else evens them out: the
  // step then takes as long as its longest tile, with most of the chip idle towards the end.)
#pragma unroll
  for (int pass = 0; pass < (PAIRED ? 2 : 1); ++pass) {
  const int tile = pass == 0 ? n_tiles - 1 - int(blockIdx.x) : int(blockIdx.x);
  if (pass == 1 && tile >= n_tiles - 1 - int(blockIdx.x)) break;   // the middle tile of an odd number is taken once
  const int seq = tiles[2 * tile], q_off = tiles[2 * tile + 1];
  // the block's HPB heads belong to one key/value head: its four-wave teams share the staged keys and values
  const int G = nq / nkv, teams_per_group = (G + HPB - 1) / HPB;
  const int g = blockIdx.y / teams_per_group, first_head = (blockIdx.y % teams_per_group) * HPB;
  const int team = threadIdx.x / (64 * WPT), wave = (threadIdx.x >> 6) % WPT, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const bool has_head = first_head + team < G;          // the last block of a group may have teams to spare
  const int h = g * G + min(first_head + team, G - 1);
  const int qlen = q_len[seq], ctx = ctx_len[seq], qs = q_start[seq];
  const int nvalid = min(16 * NQT, qlen - q_off);
  if (nvalid <= 0) continue;
  const int pos0 = ctx - qlen + q_off;
  const int k_hi = pos0 + nvalid - 1;
  const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;

  const int32_t* table = block_tables + size_t(seq) * max_blocks;
  const int first_page = k_lo >> page_shift, n_pages = (k_hi >> page_shift) - first_page + 1;
  const bool table_in_lds = n_pages <= kMaxTableLds;
  if (table_in_lds)
    for (int i = threadIdx.x; i < n_pages; i += THREADS) s_table[i] = table[first_page + i];
  // where the page numbers are read from is a compile-time choice of the caller (a run-time choice
  // between LDS and memory would turn every read into a flat load)
  auto page_at = [&](int key, auto in_lds) __attribute__((always_inline)) {
    int page;
    if constexpr (decltype(in_lds)::value) page = s_table[(key >> page_shift) - first_page];
    else page = table[key >> page_shift];
    return min(max(page, 0), num_pages - 1);
  };
  const size_t heads = size_t(nkv);
  const uint16_t* kbase = k_pool + (size_t(g) << page_shift) * HD;
  const uint16_t* vbase = v_pool + (size_t(g) << page_shift) * HD;

  bf16x8 qop[NQT][HC];
  int qpos[NQT];
  floatx4 o[NQT][DT];
  float m[NQT], lsum[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int row = 16 * qt + lr;
    const bool valid = row < nvalid;
    qpos[qt] = valid ? pos0 + row : -1;
    load_q_operand<DT>(qop[qt], valid ? q + size_t(qs + q_off + row) * q_stride + h * HD : nullptr);
    m[qt] = kNoKeyYet;
    lsum[qt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // With n_splits > 1 the stages of a tile are shared out between gridDim.z blocks, stages_per_split each
  // (the last block takes what is left, however long the sequence), and the blocks leave partial results.
  const int split = blockIdx.z;
  int range_lo = (k_lo / kStageKeys) * kStageKeys, range_hi = k_hi;
  if (n_splits > 1) {
    range_lo = max(range_lo, split * stages_per_split * kStageKeys);
    if (split + 1 < n_splits) range_hi = min(range_hi, (split + 1) * stages_per_split * kStageKeys - 1);
  }
  // A stage travels memory -> registers -> LDS.  With AHEAD the registers are asked for the next stage as soon
  // as this one lies in LDS, so its trip to memory runs while this one is being used (the registers stay
  // occupied meanwhile: worth it where there are few per thread).  (Two sets of registers, each asked for the stage
  // after the next, changed nothing: 30.6 against 30.1 us at 14 heads of 64 and 2,048 tokens.  A block does not
  // wait for its stages; its waves wait for each other at the barriers and for their own chains of dependent
  // instructions, two waves a SIMD.)
  // Which pieces of 16 bytes a thread moves.  Where the numbers divide (ROWWISE), all its key pieces lie in one key
  // row (piece kc + KT v of row kr, KT threads a row) and all its value pieces in one block of 8 keys (dims
  // vd + VD v), so that the page is looked up and the address formed once for the keys and once for the values
  // instead of once a piece: that arithmetic was a third of the vector instructions of a stage at a head size of
  // 128.  Otherwise piece threadIdx.x + THREADS u of the stage's 2 KCHUNKS, whatever it is.
  constexpr int PER_K = KCHUNKS / THREADS, PER_V = KCHUNKS / THREADS;     // keys and values hold as many pieces
  constexpr bool ROWWISE = KCHUNKS % THREADS == 0 && (HD / 8) % (PER_K > 0 ? PER_K : 1) == 0 && THREADS % 16 == 0;
  constexpr int KT = ROWWISE ? (HD / 8) / PER_K : 1, VD = THREADS / 16;
  const int kr = threadIdx.x / KT, kc = threadIdx.x % KT, vc = threadIdx.x % 16, vd = threadIdx.x / 16;
  auto fetch_from = [&](uint4 (&stage)[PER_THREAD], int key0, auto in_lds) __attribute__((always_inline)) {
    const bool interior = key0 >= k_lo && key0 + kStageKeys - 1 <= k_hi;   // no key of the stage needs clamping
    if constexpr (ROWWISE) {
      int key = key0 + kr, kb = key0 + 8 * vc;
      if (!interior) {
        key = min(max(key, k_lo), k_hi);
        kb = min(max(kb, (k_lo >> 3) << 3), (k_hi >> 3) << 3);
      }
      const uint16_t* krow = kbase + (((size_t(page_at(key, in_lds)) * heads) << page_shift) + (key & page_mask)) * HD + 8 * kc;
      const uint16_t* vcol = vbase + ((size_t(page_at(kb, in_lds)) * heads * HD + size_t(vd)) << page_shift) + (kb & page_mask);
#pragma unroll
      for (int v = 0; v < PER_K; ++v) stage[v] = ldg128(krow + 8 * KT * v);
#pragma unroll
      for (int v = 0; v < PER_V; ++v) stage[PER_K + v] = ldg128(vcol + (size_t(VD * v) << page_shift));
      return;
    }
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) {
      const int i = threadIdx.x + THREADS * u;
      if (i < KCHUNKS) {                       // keys: row r of the stage, dims 8 c .. 8 c + 7
        const int r = i / (HD / 8), c = i % (HD / 8);
        int key = key0 + r;
        if (!interior) key = min(max(key, k_lo), k_hi);
        stage[u] = ldg128(kbase + (((size_t(page_at(key, in_lds)) * heads) << page_shift) + (key & page_mask)) * HD + 8 * c);
      } else if (i < CHUNKS) {                 // values: dim d, keys 8 c .. 8 c + 7 of the stage
        const int j = i - KCHUNKS, d = j / (kStageKeys / 8), c = j % (kStageKeys / 8);
        int kb = key0 + 8 * c;
        if (!interior) kb = min(max(kb, (k_lo >> 3) << 3), (k_hi >> 3) << 3);
        stage[u] = ldg128(vbase + ((size_t(page_at(kb, in_lds)) * heads * HD + size_t(d)) << page_shift) + (kb & page_mask));
      }
    }
  };
  auto fetch = [&](uint4 (&stage)[PER_THREAD], int key0) __attribute__((always_inline)) {
    if (table_in_lds) fetch_from(stage, key0, std::true_type{});
    else fetch_from(stage, key0, std::false_type{});
  };
  // the registers of a fetched stage into LDS, between two barriers: the last stage has been used; this one is there
  auto to_lds = [&](const uint4 (&stage)[PER_THREAD]) __attribute__((always_inline)) {
    __syncthreads();
    if constexpr (ROWWISE) {
#pragma unroll
      for (int v = 0; v < PER_K; ++v) *reinterpret_cast<uint4*>(&ks[step_row(kr) * KP + 8 * (kc + KT * v)]) = stage[v];
#pragma unroll
      for (int v = 0; v < PER_V; ++v) *reinterpret_cast<uint4*>(&vs[(vd + VD * v) * VP + 8 * vc]) = stage[PER_K + v];
    } else {
#pragma unroll
      for (int u = 0; u < PER_THREAD; ++u) {
        const int i = threadIdx.x + THREADS * u;
        if (i < KCHUNKS) {
          const int r = i / (HD / 8), c = i % (HD / 8);
          *reinterpret_cast<uint4*>(&ks[step_row(r) * KP + 8 * c]) = stage[u];
        } else if (i < CHUNKS) {
          const int j = i - KCHUNKS, d = j / (kStageKeys / 8), c = j % (kStageKeys / 8);
          *reinterpret_cast<uint4*>(&vs[d * VP + 8 * c]) = stage[u];
        }
      }
    }
    __syncthreads();
  };
  // this wave's keys of the stage that lies in LDS, 32 at a time
  auto use_stage = [&](int key0) __attribute__((always_inline)) {
#pragma unroll
    for (int sub = 0; sub < WAVE_KEYS / 32; ++sub) {
      const int skey = WAVE_KEYS * wave + 32 * sub;
      const int wkey = key0 + skey;
      if (has_head && wkey <= k_hi && wkey + 32 > k_lo) {
        KVStep<DT> r;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int c = 0; c < HC; ++c) {
            const int d0 = 32 * c + 8 * lj;
            r.ka[kt][c] = d0 < HD ? as_bf16x8(*reinterpret_cast<const uint4*>(&ks[(skey + 16 * kt + lr) * KP + d0]))
                                  : as_bf16x8(make_uint4(0, 0, 0, 0));
          }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint4 v = *reinterpret_cast<const uint4*>(&vs[(16 * dt + lr) * VP + skey + 8 * lj]);
          r.va[dt][0] = make_uint2(v.x, v.y);
          r.va[dt][1] = make_uint2(v.z, v.w);
        }
        // (the unpaired block of 16 waves has no register to spare: the lazy form made it spill 36 instead of 2,
        // 529 -> 690 us for 2,048 queries over 32,768 keys; the paired one gained with it, 290 -> 264 us at 8,192)
        attend_step<DT, NQT, !(HPB * WPT == 16 && !PAIRED), true>(r, qop, o, m, lsum, wkey, k_lo, qpos, window, scale2, pos0);
      }
    }
  };
  uint4 stage[PER_THREAD];
  __syncthreads();   // the page numbers are in LDS
  if (AHEAD && range_lo <= range_hi) fetch(stage, range_lo);
  for (int key0 = range_lo; key0 <= range_hi; key0 += kStageKeys) {
    if (!AHEAD) fetch(stage, key0);
    to_lds(stage);
    if (AHEAD && key0 + kStageKeys <= range_hi) fetch(stage, key0 + kStageKeys);
    use_stage(key0);
  }

  // merge the waves of each team in turn: [wave][row][HD + 4] floats = (O^T row ..., maximum, sum, two unused).
  // A pitch of HD + 4 floats puts the 16 rows that a quarter of a wave writes or reads as 16 bytes each on
  // different LDS banks (HD + 2 with single floats collided three and four ways).
  float* mg = reinterpret_cast<float*>(smem);
  constexpr int MP = HD + 4;
#pragma unroll 1
  for (int turn = 0; turn < HPB; ++turn) {
    if (first_head + turn >= G) break;
    __syncthreads();   // the last stage, or the team before, has been read
    if (team == turn) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        float l = lsum[qt];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        float* row = mg + (size_t(wave) * 16 * NQT + 16 * qt + lr) * MP;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          *reinterpret_cast<float4*>(row + 16 * dt + 4 * lj) = make_float4(o[qt][dt][0], o[qt][dt][1], o[qt][dt][2], o[qt][dt][3]);
        if (lj == 0) { row[HD] = m[qt]; row[HD + 1] = l; }
      }
    }
    __syncthreads();
    const int head = g * G + first_head + turn;
    for (int i = threadIdx.x; i < nvalid * (HD / 4); i += THREADS) {
      const int row = i / (HD / 4), d = 4 * (i % (HD / 4));
      float mx = -INFINITY;
#pragma unroll
      for (int w = 0; w < WPT; ++w) mx = fmaxf(mx, mg[(size_t(w) * 16 * NQT + row) * MP + HD]);
      float num[4] = {0.f, 0.f, 0.f, 0.f}, den = 0.f;
#pragma unroll
      for (int w = 0; w < WPT; ++w) {
        const float* src = mg + (size_t(w) * 16 * NQT + row) * MP;
        const float f = exp2f(src[HD] - mx);
        den += f * src[HD + 1];
        const float4 part = *reinterpret_cast<const float4*>(src + d);
        num[0] += f * part.x; num[1] += f * part.y; num[2] += f * part.z; num[3] += f * part.w;
      }
      if (n_splits > 1) {
        // partial result of this block's keys: sums against the maximum mx, for the merge kernel
        const size_t slot = ((size_t(tile) * (16 * NQT) + row) * nq + head) * n_splits + split;
        *reinterpret_cast<float4*>(part_o + slot * HD + d) = make_float4(num[0], num[1], num[2], num[3]);
        if (d == 0) *reinterpret_cast<float2*>(part_ml + 2 * slot) = make_float2(mx, den);
        continue;
      }
      const float inv = den > 0.f ? 1.0f / den : 0.f;
      uint16_t* dst = out + size_t(qs + q_off + row) * (size_t(nq) * HD) + head * HD + d;
      *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(num[0] * inv, num[1] * inv), pack_bf16x2(num[2] * inv, num[3] * inv));
    }
  }
  if (PAIRED) __syncthreads();   // the merge buffer and the page numbers are free for the second tile
  }
}

// Merges the partial results of the staged kernel's key splits: one wave per (query row, head).
// part_o [tile][row][head][split][HD], part_ml [tile][row][head][split][2] = (maximum in log2 units, sum).
template <int DT, int NQT>
__global__ __launch_bounds__(256) void attention_prefill_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ tiles, uint16_t* __restrict__ out, int n_splits,
    int nq) {
  constexpr int HD = 16 * DT, ROWS = 16 * NQT;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int tile = blockIdx.x / (ROWS / 4), row = (blockIdx.x % (ROWS / 4)) * 4 + wave, h = blockIdx.y;
  const int seq = tiles[2 * tile], q_off = tiles[2 * tile + 1];
  if (q_off + row >= q_len[seq]) return;
  const size_t base = ((size_t(tile) * ROWS + row) * nq + h) * n_splits;
  float ms = kNoKeyYet, l = 0.f;
  if (lane < n_splits) {
    ms = part_ml[2 * (base + lane)];
    l = part_ml[2 * (base + lane) + 1];
  }
  const float mx = wave_max(ms);
  const float f = lane < n_splits ? exp2f(ms - mx) : 0.f;
  const float den = wave_sum(f * l);
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  uint16_t* dst = out + size_t(q_start[seq] + q_off + row) * (size_t(nq) * HD) + h * HD;
#pragma unroll
  for (int j = 0; j < (HD + 63) / 64; ++j) {
    const int d = lane + 64 * j;
    float acc = 0.f;
    for (int sp = 0; sp < n_splits; ++sp) {
      const float fs = __shfl(f, sp, 64);
      if (d < HD) acc = fmaf(fs, part_o[(base + sp) * HD + d], acc);
    }
    if (d < HD) dst[d] = f32_to_bf16_bits(acc * inv);
  }
}

// ------------------------------------------------------------------------------------------ decode
// Partial results of a block, for the merge kernel: part_o [seq][head][split][HD] (not yet divided),
// part_ml [seq][head][split][2] = (running maximum in log2 units, sum).
template <int DT, bool POW2>
__global__ __launch_bounds__(256) void attention_decode_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pool,
    const uint16_t* __restrict__ v_pool, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ decode_seqs,
    uint16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits, int nq,
    int nkv, int page_size, int num_pages, int window, float scale2) {
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2;
  __shared__ float s_o[4][16][HD + 1];
  __shared__ float s_m[4][16], s_l[4][16];
  __shared__ int32_t s_table[kDecodeChunk / 4 + 4];      // the chunk's page numbers (pages of 4 tokens or more)
  const int split = blockIdx.x, g = blockIdx.y, di = blockIdx.z;
  const int seq = decode_seqs ? decode_seqs[di] : di;   // no list: the batch is one-query sequences only, in order
  const int chunk0 = split * kDecodeChunk;
  // The page numbers of this chunk do not depend on how long the sequence is: they are asked for together with
  // its length (entries past the sequence's pages are never used), so that the keys are one trip further, not two.
  int page_shift = 0;
  if (POW2) page_shift = 31 - __builtin_clz(page_size);
  const int table_first = POW2 ? chunk0 >> page_shift : chunk0 / page_size;
  const int table_count = (POW2 ? (chunk0 + kDecodeChunk - 1) >> page_shift : (chunk0 + kDecodeChunk - 1) / page_size) - table_first + 1;
  if (int(threadIdx.x) < table_count)
    s_table[threadIdx.x] = block_tables[size_t(seq) * max_blocks + min(table_first + int(threadIdx.x), max_blocks - 1)];
  // without a list, sequence i's one query is row i
  const int q_row = decode_seqs ? q_start[seq] : seq;
  const int ctx = ctx_len[seq], pos = ctx - 1;
  const int k_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int G = nq / nkv;
  if (chunk0 > pos || chunk0 + kDecodeChunk <= k_lo) {
    // no visible key in this chunk: the merge kernel reads every chunk's (maximum, sum) without looking at
    // the context length, so an empty chunk says so itself
    if (n_splits > 1 && threadIdx.x < G) {
      const size_t slot = (size_t(di) * nq + g * G + threadIdx.x) * n_splits + split;
      part_ml[2 * slot] = kNoKeyYet;
      part_ml[2 * slot + 1] = 0.f;
    }
    return;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;

  PagedKV kv;
  kv.page_size = page_size;
  kv.num_pages = num_pages;
  kv.page_stride = size_t(nkv) * page_size * HD;
  kv.k = k_pool + size_t(g) * page_size * HD;
  kv.v = v_pool + size_t(g) * page_size * HD;
  kv.table = s_table;
  kv.table_first = table_first;
  kv.page_shift = page_shift;

  bf16x8 qop[1][HC];
  int qpos[1] = {lr < G ? pos : -1};
  load_q_operand<DT>(qop[0], lr < G ? q + size_t(q_row) * q_stride + (g * G + lr) * HD : nullptr);
  __syncthreads();   // the page numbers are in LDS
  floatx4 o[1][DT];
  float m[1] = {kNoKeyYet}, lsum[1] = {0.f};
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[0][dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // both steps of this wave are requested before the first is used
  const int w0 = chunk0 + wave * kDecodeWaveKeys;
  KVStep<DT> steps[kDecodeWaveKeys / 32];
  bool live[kDecodeWaveKeys / 32];
#pragma unroll
  for (int i = 0; i < kDecodeWaveKeys / 32; ++i) {
    const int key0 = w0 + 32 * i;
    live[i] = key0 <= pos && key0 + 32 > k_lo;
    if (live[i]) load_step<DT, POW2>(steps[i], kv, key0, k_lo, pos);
  }
#pragma unroll
  for (int i = 0; i < kDecodeWaveKeys / 32; ++i)
    if (live[i]) attend_step<DT, 1>(steps[i], qop, o, m, lsum, w0 + 32 * i, k_lo, qpos, window, scale2, pos);
  float l = lsum[0];
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (lj == 0) { s_m[wave][lr] = m[0]; s_l[wave][lr] = l; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) s_o[wave][lr][16 * dt + 4 * lj + r] = o[0][dt][r];
  __syncthreads();

  for (int i = threadIdx.x; i < G * HD; i += 256) {
    const int qh = i / HD, d = i % HD;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mx = fmaxf(mx, s_m[w][qh]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(s_m[w][qh] - mx);
      num += f * s_o[w][qh][d];
      den += f * s_l[w][qh];
    }
    const int head = g * G + qh;
    if (n_splits == 1) {
      out[size_t(q_row) * (size_t(nq) * HD) + head * HD + d] = f32_to_bf16_bits(den > 0.f ? num / den : 0.f);
    } else {
      const size_t slot = (size_t(di) * nq + head) * n_splits + split;
      part_o[slot * HD + d] = num;
      if (d == 0) { part_ml[2 * slot] = mx; part_ml[2 * slot + 1] = den; }
    }
  }
}

// Merges the chunks of one (sequence, head): grid (decode sequences, heads); lane d of a wave sums
// dimension d.  Everything a wave reads depends on its indices alone (empty chunks are marked as such by
// the decode kernel), so a wave requests 16 chunks at once: one trip to memory.  With WAVES > 1 (long
// contexts) the waves take turns of 16 chunks each and wave 0 joins their sums through LDS.
template <int DT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void attention_merge_kernel(const float* __restrict__ part_o,
                                                                     const float* __restrict__ part_ml,
                                                                     const int32_t* __restrict__ q_start,
                                                                     const int32_t* __restrict__ decode_seqs,
                                                                     uint16_t* __restrict__ out, int n_splits, int nq) {
  constexpr int HD = 16 * DT, PER_LANE = (HD + 63) / 64, GROUP = 16;
  const int di = blockIdx.x, head = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seq = decode_seqs ? decode_seqs[di] : di;
  const size_t base = (size_t(di) * nq + head) * n_splits;
  float mx = kNoKeyYet, den = 0.f, num[PER_LANE] = {};
  for (int s0 = wave * GROUP; s0 < n_splits; s0 += GROUP * WAVES) {
    float ms[GROUP], ls[GROUP], os[GROUP][PER_LANE];
#pragma unroll
    for (int i = 0; i < GROUP; ++i) {
      const bool in = s0 + i < n_splits;
      ms[i] = in ? part_ml[2 * (base + s0 + i)] : kNoKeyYet;      // the same address in every lane: one read
      ls[i] = in ? part_ml[2 * (base + s0 + i) + 1] : 0.f;
#pragma unroll
      for (int j = 0; j < PER_LANE; ++j) {
        const int d = lane + 64 * j;
        os[i][j] = (in && d < HD) ? part_o[(base + s0 + i) * HD + d] : 0.f;
      }
    }
    float group_max = mx;
#pragma unroll
    for (int i = 0; i < GROUP; ++i) group_max = fmaxf(group_max, ms[i]);
    const float keep = exp2f(mx - group_max);
    mx = group_max;
    den *= keep;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) num[j] *= keep;
#pragma unroll
    for (int i = 0; i < GROUP; ++i) {
      if (ls[i] > 0.f) {                      // an empty chunk left nothing to read in part_o
        const float f = exp2f(ms[i] - mx);
        den = fmaf(f, ls[i], den);
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) num[j] = fmaf(f, os[i][j], num[j]);
      }
    }
  }
  if constexpr (WAVES > 1) {
    __shared__ float s_mx[WAVES], s_den[WAVES], s_num[WAVES][64 * PER_LANE];
    if (lane == 0) { s_mx[wave] = mx; s_den[wave] = den; }
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) s_num[wave][lane + 64 * j] = num[j];
    __syncthreads();
    if (wave > 0) return;
    float all_max = mx;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) all_max = fmaxf(all_max, s_mx[w]);
    const float keep = exp2f(mx - all_max);
    den *= keep;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) num[j] *= keep;
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      const float f = exp2f(s_mx[w] - all_max);   // a wave without keys holds zeros: its factor does not matter
      den = fmaf(f, s_den[w], den);
#pragma unroll
      for (int j = 0; j < PER_LANE; ++j) num[j] = fmaf(f, s_num[w][lane + 64 * j], num[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < PER_LANE; ++j) {
    const int d = lane + 64 * j;
    if (d < HD)
      out[size_t(q_start[seq]) * (size_t(nq) * HD) + head * HD + d] = f32_to_bf16_bits(den > 0.f ? num[j] / den : 0.f);
  }
}

// Merge of the chunks of one head, folded into that head's share of the output projection (decode steps):
//   residual[row(di), n] += sum_d merged[di, head, d] * w_o[n, head * HD + d]
// grid (heads, blocks of 64 TPW rows of w_o, tiles of 16 TN decode sequences).  A block merges its head's chunks
// for its sequences (as attention_merge_kernel does, rounded to bfloat16 as the attention output is) into LDS,
// while its rows of w_o, requested first, are on their way; each wave then multiplies TPW tiles of 16 rows and
// adds them into the float32 residual.  Against merge kernel + projection kernel this saves a launch and the
// trip of the attention output through memory; every block of a head and a tile of sequences merges the same
// chunks again, so with many sequences a block takes more rows (TPW) and the head fewer blocks.
template <int DT, int TN, int TPW>
__global__ __launch_bounds__(256) void attention_merge_project_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ decode_seqs, const uint16_t* __restrict__ w_o, float* __restrict__ residual,
    int n_decode, int n_splits, int nq, int hidden) {
  // GROUP chunks are requested together: the 16 chunks of a context of 4,096 keys in one trip to memory
  constexpr int HD = 16 * DT, HC = (DT + 1) / 2, XP = HD + 8, GROUP = 16;
  static_assert(TN == 1, "a block merges one tile of 16 sequences");
  __shared__ __attribute__((aligned(16))) uint16_t xs[16 * TN][XP];
  __shared__ __attribute__((aligned(16))) float sums[16][64 * TPW + 4];
  __shared__ int32_t s_row[16 * TN];
  const int head = blockIdx.x, n_begin = blockIdx.y * (64 * TPW);
  const int di0 = blockIdx.z * (16 * TN);       // the block's first decode sequence
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;

  uint4 wa[TPW][HC];
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int n = min(n_begin + 16 * (wave + 4 * i) + lr, hidden - 1);
    const uint16_t* wrow = w_o + size_t(n) * (size_t(nq) * HD) + head * HD;
#pragma unroll
    for (int c = 0; c < HC; ++c) {
      const int d0 = 32 * c + 8 * lj;
      wa[i][c] = d0 < HD ? ldg128(wrow + d0) : make_uint4(0, 0, 0, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  // merge: HD / 4 threads per decode sequence, four dimensions each
  constexpr int TPR = HD / 4, ROWS = 256 / TPR;
  for (int r0 = 0; r0 < 16 * TN; r0 += ROWS) {
    const int row = r0 + int(threadIdx.x) / TPR, d = 4 * (int(threadIdx.x) % TPR);   // row of the block's tile
    if (int(threadIdx.x) >= ROWS * TPR || row >= 16 * TN) continue;
    const int di = di0 + row;
    float mx = kNoKeyYet, den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
    if (di < n_decode) {
      const size_t base = (size_t(di) * nq + head) * n_splits;
      for (int s0 = 0; s0 < n_splits; s0 += GROUP) {
        float2 ml[GROUP];
        float4 os[GROUP];
#pragma unroll
        for (int i = 0; i < GROUP; ++i) {
          const bool in = s0 + i < n_splits;
          ml[i] = in ? *reinterpret_cast<const float2*>(part_ml + 2 * (base + s0 + i)) : make_float2(kNoKeyYet, 0.f);
          // an empty chunk left nothing in part_o: its sum is zero, and what is read here is not used
          os[i] = in ? *reinterpret_cast<const float4*>(part_o + (base + s0 + i) * HD + d) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float group_max = mx;
#pragma unroll
        for (int i = 0; i < GROUP; ++i) group_max = fmaxf(group_max, ml[i].x);
        const float keep = exp2f(mx - group_max);
        mx = group_max;
        den *= keep;
#pragma unroll
        for (int r = 0; r < 4; ++r) num[r] *= keep;
#pragma unroll
        for (int i = 0; i < GROUP; ++i) {
          if (ml[i].y > 0.f) {
            const float f = exp2f(ml[i].x - mx);
            den = fmaf(f, ml[i].y, den);
            num[0] = fmaf(f, os[i].x, num[0]);
            num[1] = fmaf(f, os[i].y, num[1]);
            num[2] = fmaf(f, os[i].z, num[2]);
            num[3] = fmaf(f, os[i].w, num[3]);
          }
        }
      }
      if (d == 0) s_row[row] = q_start[decode_seqs ? decode_seqs[di] : di];
    }
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    *reinterpret_cast<uint2*>(&xs[row][d]) = make_uint2(pack_bf16x2(num[0] * inv, num[1] * inv), pack_bf16x2(num[2] * inv, num[3] * inv));
  }
  __syncthreads();

  // The sums go through LDS so that a wave adds 64 neighbouring numbers of one sequence's row of the residual at a
  // time: heads add into the same rows, and atomics scattered over 16 rows a wave take many times longer.
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int tile = wave + 4 * i;
    if (n_begin + 16 * tile >= hidden || di0 >= n_decode) continue;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < HC; ++c) {
      const int d0 = 32 * c + 8 * lj;
      const uint4 b = d0 < HD ? *reinterpret_cast<const uint4*>(&xs[lr][d0]) : make_uint4(0, 0, 0, 0);
      acc = mfma16(as_bf16x8(wa[i][c]), as_bf16x8(b), acc);
    }
    // lane holds rows 16 tile + 4 lj + 0..3 of the block's rows of w_o for sequence di0 + lr
    *reinterpret_cast<float4*>(&sums[lr][16 * tile + 4 * lj]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 16 * 64 * TPW; i += 256) {
    const int t = i / (64 * TPW), n = n_begin + i % (64 * TPW);
    if (di0 + t < n_decode && n < hidden) unsafeAtomicAdd(residual + size_t(s_row[t]) * hidden + n, sums[t][i % (64 * TPW)]);
  }
}

// ------------------------------------------------------------------------------------------ host side
bool attention_mfma_supports(int hd, int page_size, int nq, int nkv) {
  const int dt = hd / 16;
  const bool hd_ok = hd % 16 == 0 && (dt <= 6 || dt == 8);
  return hd_ok && page_size % 4 == 0;
}
bool attention_mfma_decode_supports(int nq, int nkv) { return nq / nkv <= 16; }
int attention_mfma_tile_q(int hd) { return 32; }

constexpr int kMaxPrefillSplits = 32;   // the merge kernel holds one split per lane; 64 would do as well

static bool staged_prefill(int page_size) { return page_size >= 8 && (page_size & (page_size - 1)) == 0; }

// Blocks per tile and head along the keys.  A step with few queries over a long context (a portion of a long
// prompt) has few tiles, each with a long walk: the walk is cut until the grid fills the chip about three times.
// Teams of a block of the staged kernel: HPB heads of one key/value head, WPT waves each.  The heads share
// every stage of keys and values, which the kernel otherwise fetches from L2 once per head -- and that
// traffic, not the matrix cores, is what bounds it (measured ~8.5 TB/s at every size).  Head sizes up to 64:
// four teams of four waves.  Above that the registers of 16 waves do not suffice: four teams of two waves
// (each wave then takes 64 keys of a stage).  Three teams were slower than two or four at every size.
// A portion of 2,048 tokens at a context of 32,768: 835 -> 472 us (14 heads of 64), 2,350 -> 1,470 us (28 of 128).
struct StagedShape { int hpb, wpt; bool ahead; };
static StagedShape staged_shape(int nq, int nkv, int hd, int n_tiles) {
  const int G = nq / nkv;
  if (G <= 1) return {1, 4, false};
  if (G == 2) return {2, 4, hd > 64};
  if (hd > 64) return {4, 2, false};
  // Head sizes up to 64: four heads a block stage every key once for four heads, but a portion of a prompt has
  // few tiles, and four heads a block then leave most CUs without one.  As many heads a block as still give every
  // CU a block (14 heads of 64 in 2 groups, time to the first token over 4 layers: 4,096 tokens in portions of
  // 256: 4.88 ms with four heads a block, 4.80 with two, 4.62 with one; 8,192 in portions of 1,024: 5.64, 5.05,
  // 5.47; 2,048 at once: 1.07, 1.16, 1.09; 16,384 in portions of 2,048: 9.38, 10.76, 11.42).  At a head size of
  // 128 the block of four heads on two waves each was the fastest at every portion size.
  if (n_tiles * nkv * ((G + 3) / 4) >= 256) return {4, 4, true};
  if (n_tiles * nkv * ((G + 1) / 2) >= 256) return {2, 4, false};
  return {1, 4, false};
}
// Whether the tiles are taken in pairs (a long walk and a short one per block), and with which teams.
static bool staged_paired(int n_tiles, int nq, int nkv, int hd, int splits, int max_tile_ctx, int mean_tile_walk,
                          StagedShape* shape) {
  // Measured (one causal prompt, kernel time in us, unpaired -> paired): 28 heads of 128 in 4 groups, 2,048 tokens
  // 112 -> 73, 16,384 tokens 3,240 -> 3,140, a portion of 2,048 after 8,192 earlier tokens 519 -> 503; 16 heads of
  // 64 in 8 groups, 2,048 tokens 57 -> 34.  With fewer pairs than CUs, halving the number of blocks costs more
  // than the even walks gain.
  const int G = nq / nkv;
  if (splits > 1 || n_tiles < 2) return false;
  const int pairs = (n_tiles + 1) / 2;
  if (pairs * nkv * ((G + shape->hpb - 1) / shape->hpb) >= 256) return true;
  // Teams of 16 waves: two heads a block instead of four make twice the blocks, but fetch every stage twice
  // as often.  That pays only while the walks differ much: the longest at least 1.5 times the mean, as in a prompt's
  // first portion (14 heads of 64 in 2 groups, 2,048 tokens: 39.5 -> 33.5 after no earlier tokens, 55.7 -> 55.7
  // after 1,024, 72 -> 79 after 2,048).
  if (hd <= 64 && shape->hpb == 4 && pairs * nkv * ((G + 1) / 2) >= 256 && 3 * mean_tile_walk <= 2 * max_tile_ctx) {
    *shape = StagedShape{2, 4, true};
    return true;
  }
  return false;
}

int attention_prefill_splits(int n_tiles, int nq, int nkv, int hd, int page_size, int max_tile_ctx) {
  if (!staged_prefill(page_size)) return 1;
  const StagedShape shape = staged_shape(nq, nkv, hd, n_tiles);
  const int G = nq / nkv;
  const int blocks = n_tiles * nkv * ((G + shape.hpb - 1) / shape.hpb), stages = (max_tile_ctx + kStageKeys - 1) / kStageKeys;
  const int enough = 2048 / (shape.wpt * shape.hpb);   // blocks that hold 2,048 waves: two rounds of the chip's CUs
  if (blocks <= 0 || blocks >= enough || stages <= 4) return 1;
  return max(1, min(min((enough * 3 / 2 + blocks - 1) / blocks, stages / 2), kMaxPrefillSplits));
}

size_t attention_prefill_workspace_floats(int n_tiles, int nq, int nkv, int hd, int page_size, int max_tile_ctx) {
  const size_t splits = attention_prefill_splits(n_tiles, nq, nkv, hd, page_size, max_tile_ctx);
  return splits <= 1 ? 0 : size_t(n_tiles) * 32 * nq * splits * (hd + 2);
}

size_t attention_decode_workspace_floats(int n_decode, int nq, int hd, int max_ctx) {
  const size_t splits = (max_ctx + kDecodeChunk - 1) / kDecodeChunk;
  return splits <= 1 ? 0 : size_t(n_decode) * nq * splits * (hd + 2);
}

template <int DT>
static int launch_mfma(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                       const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                       const int32_t* ctx_len, const int32_t* tiles, int n_tiles, const int32_t* decode_seqs,
                       int n_decode, int max_decode_ctx, int max_tile_ctx, int mean_tile_walk, float* workspace,
                       void* out, int nq, int nkv, int page_size, int num_pages, int window, float scale) {
  constexpr int HD = 16 * DT;
  constexpr int NQT = 2;
  const float scale2 = scale * kLog2e;
  const uint16_t *qp = (const uint16_t*)q, *kp = (const uint16_t*)k_pool, *vp = (const uint16_t*)v_pool;
  // the workspace holds the decode partials first, then the prefill partials
  float* prefill_ws = workspace ? workspace + attention_decode_workspace_floats(n_decode, nq, HD, max_decode_ctx) : nullptr;
  if (n_tiles > 0) {
    if (staged_prefill(page_size)) {
      int page_shift = 0;
      while ((1 << page_shift) < page_size) ++page_shift;
      const int splits = attention_prefill_splits(n_tiles, nq, nkv, HD, page_size, max_tile_ctx);
      const int stages = (max_tile_ctx + kStageKeys - 1) / kStageKeys;
      const int per_split = (stages + splits - 1) / splits;
      float* part_o = splits > 1 ? prefill_ws : nullptr;
      float* part_ml = splits > 1 ? prefill_ws + size_t(n_tiles) * 16 * NQT * nq * splits * HD : nullptr;
      StagedShape shape = staged_shape(nq, nkv, HD, n_tiles);
      const bool paired = staged_paired(n_tiles, nq, nkv, HD, splits, max_tile_ctx, mean_tile_walk, &shape);
      const dim3 grid(paired ? (n_tiles + 1) / 2 : n_tiles, nkv * ((nq / nkv + shape.hpb - 1) / shape.hpb), splits);
#define SP_STAGED(HPB, WPT, AHEAD, PAIRED)                                                                      \
  attention_prefill_staged_kernel<DT, NQT, HPB, WPT, AHEAD, PAIRED><<<grid, 64 * WPT * HPB, 0, s>>>(            \
      qp, q_stride, kp, vp, block_tables, max_blocks, q_start, q_len, ctx_len, tiles, (uint16_t*)out, part_o,   \
      part_ml, splits, per_split, nq, nkv, page_shift, num_pages, window, scale2, n_tiles)
      // the same cases as staged_shape() and staged_paired()
      if (paired) {
        if (shape.hpb == 1) SP_STAGED(1, 4, false, true);
        else if (shape.hpb == 2) SP_STAGED(2, 4, true, true);
        else { if constexpr (DT > 4) SP_STAGED(4, 2, false, true); else SP_STAGED(4, 4, true, true); }
      }
      else if (shape.hpb == 1) SP_STAGED(1, 4, false, false);
      else if (shape.hpb == 2) { if constexpr (DT > 4) SP_STAGED(2, 4, true, false); else SP_STAGED(2, 4, false, false); }
      else { if constexpr (DT > 4) SP_STAGED(4, 2, false, false); else SP_STAGED(4, 4, true, false); }
#undef SP_STAGED
      if (splits > 1) {
        if (check_launch("sp_attention (prefill)")) return 1;
        attention_prefill_merge_kernel<DT, NQT><<<dim3(n_tiles * (16 * NQT / 4), nq), 256, 0, s>>>(
            part_o, part_ml, q_start, q_len, tiles, (uint16_t*)out, splits, nq);
      }
    } else {
      attention_prefill_kernel<DT, NQT><<<dim3(n_tiles, nq), 64, 0, s>>>(
          qp, q_stride, kp, vp, block_tables, max_blocks, q_start, q_len, ctx_len, tiles, (uint16_t*)out, nq, nkv,
          page_size, num_pages, window, scale2);
    }
    if (check_launch("sp_attention (prefill)")) return 1;
  }
  if (n_decode > 0) {
    const int n_splits = max(1, (max_decode_ctx + kDecodeChunk - 1) / kDecodeChunk);
    float* part_o = workspace;
    float* part_ml = workspace ? workspace + size_t(n_decode) * nq * n_splits * HD : nullptr;
    if ((page_size & (page_size - 1)) == 0)
      attention_decode_kernel<DT, true><<<dim3(n_splits, nkv, n_decode), 256, 0, s>>>(
          qp, q_stride, kp, vp, block_tables, max_blocks, q_start, ctx_len, decode_seqs, (uint16_t*)out, part_o, part_ml,
          n_splits, nq, nkv, page_size, num_pages, window, scale2);
    else
      attention_decode_kernel<DT, false><<<dim3(n_splits, nkv, n_decode), 256, 0, s>>>(
          qp, q_stride, kp, vp, block_tables, max_blocks, q_start, ctx_len, decode_seqs, (uint16_t*)out, part_o, part_ml,
          n_splits, nq, nkv, page_size, num_pages, window, scale2);
    if (check_launch("sp_attention (decode)")) return 1;
    if (n_splits > 1) {
      if (n_splits <= 16)
        attention_merge_kernel<DT, 1><<<dim3(n_decode, nq), 64, 0, s>>>(part_o, part_ml, q_start, decode_seqs,
                                                                         (uint16_t*)out, n_splits, nq);
      else
        attention_merge_kernel<DT, 4><<<dim3(n_decode, nq), 256, 0, s>>>(part_o, part_ml, q_start, decode_seqs,
                                                                          (uint16_t*)out, n_splits, nq);
      if (check_launch("sp_attention (merge)")) return 1;
    }
  }
  return 0;
}

int attention_mfma(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                   const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                   const int32_t* ctx_len, const int32_t* tiles, int n_tiles, const int32_t* decode_seqs, int n_decode,
                   int max_decode_ctx, int max_tile_ctx, int mean_tile_walk, float* workspace, void* out, int nq, int nkv,
                   int hd, int page_size, int num_pages, int window, float scale) {
#define SP_MFMA(DT)                                                                                              \
  case DT:                                                                                                       \
    return launch_mfma<DT>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len, ctx_len,    \
                           tiles, n_tiles, decode_seqs, n_decode, max_decode_ctx, max_tile_ctx, mean_tile_walk,  \
                           workspace, out, nq, nkv, page_size, num_pages, window, scale)
  switch (hd / 16) {
    SP_MFMA(1); SP_MFMA(2); SP_MFMA(3); SP_MFMA(4); SP_MFMA(5); SP_MFMA(6); SP_MFMA(8);
  }
#undef SP_MFMA
  set_error("sp_attention: no matrix-core kernel for head size %d", hd);
  return 1;
}

// Decode steps whose chunks' merge is folded into the output projection.  Worth it where the merged partial
// results, which every block of a head and a tile of 16 sequences reads again, stay small beside the rows of w_o
// (measured at 14 heads of 64, a width of 896, contexts of 4,096, tokens a second with the fold against merge and
// projection kernels of their own: 8 sequences 8,250 against 7,930, 24 sequences 21,870 against 21,260, 32
// sequences 27,400 against 26,660, 64 sequences 39,840 against 40,350).
bool attention_decode_project_takes(int hd, int page_size, int nq, int nkv, int n_decode, int max_decode_ctx, int hidden) {
  if (!attention_mfma_supports(hd, page_size, nq, nkv) || !attention_mfma_decode_supports(nq, nkv)) return false;
  const int n_splits = (max_decode_ctx + kDecodeChunk - 1) / kDecodeChunk;
  return n_decode >= 1 && n_decode <= 32 && n_splits > 1 && min(n_decode, 16) * n_splits <= 256 && hidden >= 16 &&
         hidden <= 2048;   // (wider: 28 heads of 128 at 3,584 +1%, 40 heads at 5,120 -0.5% with four tiles a wave)
}

// Tiles of 16 rows of w_o a wave takes in the folded kernel: one up to 16 sequences; with more, every tile of 16
// sequences is a block of its own and merges the head's chunks again, so a block takes as many rows as still
// leaves about 200 blocks (24 and 32 sequences, 14 heads, a width of 896: two tiles a wave 21,870 and 27,400
// tokens a second, one 21,600 and 27,100, four 21,400 and 26,990).
static int project_tiles_per_wave(int n_decode, int nq, int hidden) {
  if (n_decode <= 16) return 1;
  const int seq_tiles = (n_decode + 15) / 16;
  for (int tpw = 4; tpw > 1; tpw /= 2)
    if (nq * ((hidden + 64 * tpw - 1) / (64 * tpw)) * seq_tiles >= 192) return tpw;
  return 1;
}

template <int DT>
static int launch_decode_project(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                 const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                                 const int32_t* ctx_len, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                                 float* workspace, const void* w_o, float* residual, int hidden, int nq, int nkv,
                                 int page_size, int num_pages, int window, float scale) {
  constexpr int HD = 16 * DT;
  const int n_splits = (max_decode_ctx + kDecodeChunk - 1) / kDecodeChunk;
  float* part_o = workspace;
  float* part_ml = workspace + size_t(n_decode) * nq * n_splits * HD;
  if ((page_size & (page_size - 1)) == 0)
    attention_decode_kernel<DT, true><<<dim3(n_splits, nkv, n_decode), 256, 0, s>>>(
        (const uint16_t*)q, q_stride, (const uint16_t*)k_pool, (const uint16_t*)v_pool, block_tables, max_blocks, q_start,
        ctx_len, decode_seqs, nullptr, part_o, part_ml, n_splits, nq, nkv, page_size, num_pages, window, scale * kLog2e);
  else
    attention_decode_kernel<DT, false><<<dim3(n_splits, nkv, n_decode), 256, 0, s>>>(
        (const uint16_t*)q, q_stride, (const uint16_t*)k_pool, (const uint16_t*)v_pool, block_tables, max_blocks, q_start,
        ctx_len, decode_seqs, nullptr, part_o, part_ml, n_splits, nq, nkv, page_size, num_pages, window, scale * kLog2e);
  if (check_launch("sp_attention_decode_project (decode)")) return 1;
  const int tpw = project_tiles_per_wave(n_decode, nq, hidden);
  const dim3 grid(nq, (hidden + 64 * tpw - 1) / (64 * tpw), (n_decode + 15) / 16);
#define SP_PROJECT(TPW)                                                                                         \
  attention_merge_project_kernel<DT, 1, TPW><<<grid, 256, 0, s>>>(part_o, part_ml, q_start, decode_seqs,        \
                                                                   (const uint16_t*)w_o, residual, n_decode,     \
                                                                   n_splits, nq, hidden)
  if (tpw == 1) SP_PROJECT(1);
  else if (tpw == 2) SP_PROJECT(2);
  else SP_PROJECT(4);
#undef SP_PROJECT
  return check_launch("sp_attention_decode_project (merge and projection)");
}

int attention_mfma_decode_project(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                  const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                                  const int32_t* ctx_len, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                                  float* workspace, const void* w_o, float* residual, int hidden, int nq, int nkv,
                                  int hd, int page_size, int num_pages, int window, float scale) {
#define SP_MFMA(DT)                                                                                              \
  case DT:                                                                                                       \
    return launch_decode_project<DT>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, ctx_len, \
                                     decode_seqs, n_decode, max_decode_ctx, workspace, w_o, residual, hidden,    \
                                     nq, nkv, page_size, num_pages, window, scale)
  switch (hd / 16) {
    SP_MFMA(1); SP_MFMA(2); SP_MFMA(3); SP_MFMA(4); SP_MFMA(5); SP_MFMA(6); SP_MFMA(8);
  }
#undef SP_MFMA
  set_error("sp_attention_decode_project: no matrix-core kernel for head size %d", hd);
  return 1;
}

}  // namespace sprout
