// Gather-rows GEMM that streams both operands through LDS with direct-to-LDS buffer loads, for
// contractions that fit one channel chunk (see rowgemm.h for the problem statement).
//
// Why: in the register-gather kernels a lane loads the 16 bytes its MFMA operand slot needs, so
// neighbouring lanes read different rows and every load instruction is 64 separate 16-byte
// requests; and the step body spends most of its issue slots on addressing, descriptor selection
// and LDS staging of the weights.  Here
//   * a load instruction moves whole rows: 4*KS neighbouring lanes read one row's KS*64 bytes
//     (one request per 64-byte segment), and the data lands in LDS without passing registers
//     (buffer_load ... lds writes lane l of the instruction at M0 + 16*l);
//   * the LDS image of a tile is row-major with the 16-byte chunks of a row XOR-permuted by
//     swz(row) = (row*KS/4) mod 4*KS ((row/2) mod 4 for 64-byte rows, two of which share a
//     128-byte line of banks).  The permutation is applied on the global side (a lane picks
//     which chunk of its row it fetches), which keeps the global access coalesced, and makes the
//     MFMA-layout reads (16 lanes = 16 rows, same chunk) hit 16 different bank groups;
//   * the weight tile is stored in the row order the MFMA fragments want (LDS row wn*NBW*16 +
//     nb*16 + i holds output channel wn*NBW*16 + (i/4)*4*NBW + nb*4 + i%4), so that a lane's
//     accumulators are 4*NBW consecutive channels of one output row (vector stores, no atomics);
//   * waves form a WM x WN grid over the tile; each wave reads RBW row fragments and NBW weight
//     fragments per 16-byte k-step from LDS, i.e. (WM*TN + WN*TM)*KS*64 bytes per offset instead
//     of NW*TN*KS*64;
//   * NS stages of (rows + weights) form a ring; one barrier per kernel offset.  Step i waits for
//     its own loads of offset i, passes the barrier (now everybody's loads of offset i have landed
//     and everybody has finished computing offset i-1), issues the loads of offset i+NS-1 into the
//     stage that offset i-1 used, then computes.  Pair-table entries run NS steps ahead of the row
//     loads that need them.  A kernel offset past the end of the tile's list is loaded through a
//     descriptor with zero records (no memory traffic, zeros into LDS), which keeps the number of
//     outstanding loads the same on every path: the waits below count instructions.
//   * every stage is its own __shared__ array: the compiler then knows which direct-to-LDS loads
//     an LDS read can depend on and does not wait for the younger ones.
#pragma once
#include <type_traits>
#include <utility>

#include "lds_dma.h"
#include "rowgemm.h"

namespace cummhip {

template <class F, int... Is>
__device__ __forceinline__ bool run_steps(F &f, std::integer_sequence<int, Is...>) {
  return (f(std::integral_constant<int, Is>{}) || ...);
}

// T: element tag; WM x WN: wave grid; RBW: 16-row blocks per wave; NBW: 16-channel blocks per
// wave; KS: 64-byte pieces per row (contraction <= KS*64 bytes); NS: ring stages.
// WT false: weights are contiguous along the contraction (w_stride_c == 1).
// WT true (two-byte elements): weights are contiguous along the output channel (w_stride_n == 1).
// The weight tile then sits in LDS as [contraction][channel] rows, again with XOR-permuted
// 16-byte chunks, and the MFMA operand is fetched with the transposing LDS read: within a group
// of 16 lanes, ds_read_b64_tr_b16 hands lane i, element j the 16-bit element i%4 of the 8 bytes
// that lane i/4 + 4j points to.  Lane s of a group points to row (first k) + s/4, channels
// 4*(s%4) .. +3 of its 16-channel block, so lane i receives 4 consecutive k of channel i; two
// reads make one operand.  A lane then owns channels nb*16 + 4q .. +3 of each block nb.
// WIDE: four-byte outputs (s32 / f32: the accumulators through the linear combination, see
// store_wide_piece in rowgemm.h).
// The LDS a tile body works in: row part and weight part of each ring stage, and the slots of the
// pair-table entries.  The kernels below declare the arrays (every stage its own __shared__ array,
// see above) and hand them over; the body is inlined, so these are compile-time addresses.
struct LdsRing {
  v4i *rows[4];
  v4i *weights[4];
  int (*idx[4])[64];
};

// One tile: rows [tile * TM, tile * TM + TM) of the sorted positions, column block col.
// HALVES: mask_out takes one word per 64 positions (a 128-row tile writes words 2 tile, 2 tile + 1).
// HALF32 (TM = 32): the tile is one half of a 64-row tile, whose word of mask_out (the OR over
// all 64 positions, written by the even half) and whose skip rule (left alone only if the whole
// 64-row tile has no offset) it keeps, so that the launch gives what 64-row tiles give.
// MW: 32-bit mask words per position.  1 = one word (kernel volumes up to 32).  4 = the layout
// of the reference's dynamic-mask kernels for larger volumes (MaskIGemmIteratorMaskLoaderDynamic,
// cumm/gemm/blockmma/mma.py:78-269): p.mask_words = ceil(kv / 32) words per position, word w of
// position pos at mask[pos * mask_words + w] holding offsets 32 w .. 32 w + 31; mask_out likewise
// per tile; the filter applies to every word.
template <class T, int WM, int WN, int RBW, int NBW, int KS, int NS, bool WT, bool WIDE, bool HALVES, int MW = 1, bool HALF32 = false>
__device__ __forceinline__ void rowgemm_lds_tile(const RowGemmParams &p, const int tile, const int col, const LdsRing &lds) {
  static_assert(MW == 1 || MW == 4, "one mask word, or up to four");
  static_assert(MW == 1 || (!HALVES && !HALF32), "the tile shapes of a mixed launch take one mask word");
  static_assert(!HALF32 || (WM * RBW * 16 == 32 && !HALVES), "a half of a 64-row tile has 32 rows");
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr int TM = WM * RBW * 16;
  constexpr int TN = WN * NBW * 16;
  constexpr int PV = E::kPerVec;
  constexpr int LPR = 4 * KS;              // lanes (16-byte chunks) per row
  constexpr int RPI = 64 / LPR;            // rows per load instruction
  constexpr int IPA = TM * LPR / NT;       // row-load instructions per wave and offset
  constexpr int IPW = TN * LPR / NT;       // weight-load instructions per wave and offset
  // transposed weight tile: KS*64/kBytes rows of TN elements
  constexpr int WROWS = KS * 64 / E::kBytes;         // contraction rows
  constexpr int LPRW = TN * E::kBytes / 16;          // lanes (16-byte chunks) per row
  constexpr int RPIW = 64 / LPRW;                    // rows per load instruction
  static_assert(!WT || E::kBytes == 2, "the transposing read used here moves 16-bit elements");
  static_assert(!WT || WROWS * LPRW == TN * LPR, "both weight layouts fill the same LDS bytes");
  static_assert(IPA >= 1 && IPW >= 1, "tile too small for the workgroup");
  constexpr int A_V = TM * LPR;            // 16-byte vectors of the row part of a stage
  constexpr int STAGE_V = (TM + TN) * LPR;
  constexpr int L = NS - 1;                // steps the operand loads run ahead
  constexpr int DI = NS;                   // steps the pair-table loads run ahead of the row loads
  constexpr int RPW = TM / NW;             // rows whose entries a wave fetches (one instruction)
  static_assert(RPW <= 64, "one entry instruction per wave");
  constexpr int PER_STEP = IPA + IPW + 1;  // load instructions a wave issues per step
  // loads issued after those of offset i when step i starts: the entries issued with them, then
  // L-1 whole steps
  constexpr int WAIT_OPERANDS = 1 + (L - 1) * PER_STEP;
  static_assert(WAIT_OPERANDS < 64, "too many loads in flight for the counter");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int m = lane & 15;
  const int q = lane >> 4;
  auto stage = [&](auto sc) -> v4i * { return lds.rows[decltype(sc)::value]; };
  auto stage_w = [&](auto sc) -> v4i * { return lds.weights[decltype(sc)::value]; };
  auto idx_slot = [&](auto sc) -> int * { return lds.idx[decltype(sc)::value][wave]; };

  const int n0 = col * TN;
  const int pos_base = tile * TM;

  // ---- the tile's mask words are requested first and reduced only after the row keys below have
  // been requested too: one memory round trip for both
  // All per-position loads of this prologue (mask words, row keys, output rows) are issued first,
  // back to back, as hidden buffer loads through descriptors that end at n_pos (no records when
  // the array is absent: a position past the end reads 0), then waited for once; the values are
  // chosen afterwards with selects.  Written as conditional C++ loads, every one of them was
  // compiled into a branch with a wait of its own behind it and the prologue paid four to five
  // dependent round trips (1.3 us of a one-offset tile's 3.8) instead of one.
  const bool has_mask = p.mask != nullptr;
  const bool has_rows = p.out_rows != nullptr;
  const int mic = MW == 1 ? 1 : p.mask_words;     // words per position actually there
  const v4i rsw_mask = rsrc_words(p.mask, has_mask ? (uint32_t)p.n_pos * 4u * (uint32_t)mic : 0u);
  // byte offset of word w of a position's mask (pos_off of the position given)
  auto word_off = [&](uint32_t pos_off4, int w) __attribute__((always_inline)) -> uint32_t {
    if constexpr (MW == 1) return pos_off4;
    else return pos_off4 != kOob && w < mic ? pos_off4 * (uint32_t)mic + 4u * (uint32_t)w : kOob;
  };
  const v4i rsw_rows = rsrc_words(p.out_rows, has_rows ? (uint32_t)p.n_pos * 4u : 0u);
  auto pos_off = [&](int pos) __attribute__((always_inline)) -> uint32_t { return pos >= 0 && pos < p.n_pos ? (uint32_t)pos * 4u : kOob; };
  constexpr int MKW = (TM + 63) / 64;
  const int lrow = lane / LPR;             // row inside a load instruction
  const int lchunk = lane % LPR;           // LDS chunk slot inside the row
  const int key_pos = pos_base + wave * RPW + lane;   // entries: lane l < RPW fetches the entry of row wave*RPW + l
  int raw_mk[MKW][MW], raw_key_row, raw_key_bits[MW], raw_a_row[IPA], raw_a_bits[IPA][MW], raw_o_row[RBW];
#pragma unroll
  for (int i = 0; i < MKW; ++i)
#pragma unroll
    for (int w = 0; w < MW; ++w)
      raw_mk[i][w] = load_b32_hidden(rsw_mask, word_off(i * 64 + lane < TM ? pos_off(pos_base + i * 64 + lane) : kOob, w));
  // HALF32: the masks of the other half of the 64-row tile (lanes 0 .. 31)
  int raw_other = 0;
  if constexpr (HALF32) raw_other = load_b32_hidden(rsw_mask, lane < 32 ? pos_off((pos_base ^ 32) + lane) : kOob);
  raw_key_row = load_b32_hidden(rsw_rows, pos_off(key_pos));
#pragma unroll
  for (int w = 0; w < MW; ++w) raw_key_bits[w] = load_b32_hidden(rsw_mask, word_off(pos_off(key_pos), w));
#pragma unroll
  for (int t = 0; t < IPA; ++t) {
    const int pos = pos_base + (wave * IPA + t) * RPI + lrow;
    raw_a_row[t] = load_b32_hidden(rsw_rows, pos_off(pos));
#pragma unroll
    for (int w = 0; w < MW; ++w) raw_a_bits[t][w] = load_b32_hidden(rsw_mask, word_off(pos_off(pos), w));
  }
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
    raw_o_row[rb] = load_b32_hidden(rsw_rows, pos_off(pos_base + (wm * RBW + rb) * 16 + m));
  // requantisation scale and bias of this lane's output channels (one-byte outputs): requested
  // behind the masks and keys and landing with them; without the int8 epilogue the descriptors
  // have no records
  float scale_v[E::kBytes == 1 ? 4 * NBW : 1], bias_v[E::kBytes == 1 ? 4 * NBW : 1];
  if constexpr (E::kBytes == 1) {
    const uint32_t sb_bytes = p.int8_epilogue ? (uint32_t)p.k_out * 4u : 0u;
    const __amdgpu_buffer_rsrc_t rs_scale = make_rsrc(p.scale, sb_bytes);
    const __amdgpu_buffer_rsrc_t rs_bias = make_rsrc(p.bias, sb_bytes);
    const uint32_t off = (uint32_t)(n0 + wn * (NBW * 16) + q * (4 * NBW)) * 4u;
#pragma unroll
    for (int g = 0; g < NBW; ++g) {
      // (whole-vector casts: a per-element cast of the loaded vector was seen to be compiled
      // into a load of element 0 only)
      const v4f sv = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs_scale, off + g * 16, 0, 0));
      const v4f bv = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rs_bias, off + g * 16, 0, 0));
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        scale_v[g * 4 + x] = sv[x];
        bias_v[g * 4 + x] = bv[x];
      }
    }
  }

  wait_vmcnt<0>();
#pragma unroll
  for (int i = 0; i < MKW; ++i)
#pragma unroll
    for (int w = 0; w < MW; ++w) keep_after_wait(raw_mk[i][w]);
  if constexpr (HALF32) keep_after_wait(raw_other);
  keep_after_wait(raw_key_row);
#pragma unroll
  for (int w = 0; w < MW; ++w) keep_after_wait(raw_key_bits[w]);
#pragma unroll
  for (int t = 0; t < IPA; ++t) {
    keep_after_wait(raw_a_row[t]);
#pragma unroll
    for (int w = 0; w < MW; ++w) keep_after_wait(raw_a_bits[t][w]);
  }
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) keep_after_wait(raw_o_row[rb]);
  uint32_t mk[MW];
#pragma unroll
  for (int w = 0; w < MW; ++w) {
    mk[w] = 0;
#pragma unroll
    for (int i = 0; i < MKW; ++i) mk[w] |= (uint32_t)raw_mk[i][w];
  }

  // ---- loader role of this lane: rows of the tile it fetches, weight rows it fetches
  auto swz = [](int row) { return KS == 1 ? (row >> 1) & 3 : ((row * KS) >> 2) & (LPR - 1); };
  const bool has_gather = p.gather != nullptr;
  // entries: lane l < RPW fetches the entry of tile row wave*RPW + l
  // A row takes part in kernel offset k only if its own mask word has the bit (the word is
  // what the pair table was built from: bit clear = entry -1).  Entries and rows of the others
  // are not fetched at all: the 4-byte entries are scattered over the table, one memory sector
  // each, and on sparse offsets most rows of a tile have none.
  auto row_bits = [&](int raw) __attribute__((always_inline)) -> uint32_t {
    const uint32_t w = (uint32_t)raw;
    const uint32_t wr = __builtin_bitreverse32(w) >> ((32 - p.kv) & 31);
    return has_mask && !p.ungated_rows ? (p.reverse_mask ? wr : w) : ~0u;
  };
  // The same for MW words: the kv-bit string over the words reversed end for end (bit j of the
  // result = bit kv-1-j), as the reference's loader walks a reversed mask (mma.py:196-215).
  // (The words of a row are one vector value, not an array: an array that is indexed through a
  // select ends up in scratch memory, whose accesses would count in vmcnt.)
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  using Words = std::conditional_t<MW == 1, uint32_t, v4u>;
  auto reverse_words = [&](const v4u m) __attribute__((always_inline)) -> v4u {
    const int s = (mic * 32 - p.kv) & 31;     // unused bits at the top of the last word
    const uint32_t b0 = __builtin_bitreverse32(m[0]), b1 = __builtin_bitreverse32(m[1]);
    const uint32_t b2 = __builtin_bitreverse32(m[2]), b3 = __builtin_bitreverse32(m[3]);
    // word i of the reversed string before the shift = reversed word mic-1-i
    v4u r;
    r[0] = mic == 4 ? b3 : (mic == 3 ? b2 : (mic == 2 ? b1 : b0));
    r[1] = mic == 4 ? b2 : (mic == 3 ? b1 : (mic == 2 ? b0 : 0u));
    r[2] = mic == 4 ? b1 : (mic == 3 ? b0 : 0u);
    r[3] = mic == 4 ? b0 : 0u;
    if (s == 0) return r;
    v4u o;
    o[0] = (r[0] >> s) | (r[1] << (32 - s));
    o[1] = (r[1] >> s) | (r[2] << (32 - s));
    o[2] = (r[2] >> s) | (r[3] << (32 - s));
    o[3] = r[3] >> s;
    return o;
  };
  auto row_words = [&](const int (&raw)[MW]) __attribute__((always_inline)) -> Words {
    if constexpr (MW == 1) {
      return row_bits(raw[0]);
    } else {
      v4u m = {(uint32_t)raw[0], (uint32_t)raw[1], (uint32_t)raw[2], (uint32_t)raw[3]};
      if (p.reverse_mask) m = reverse_words(m);
      if (!has_mask || p.ungated_rows) m = v4u{~0u, ~0u, ~0u, ~0u};
      return m;
    }
  };
  // bit k of a row's words (k wave-uniform; k < 0 comes with a descriptor without records)
  auto has_bit = [&](const Words m, int k) __attribute__((always_inline)) -> uint32_t {
    if constexpr (MW == 1) {
      return (m >> (k & 31)) & 1u;
    } else {
      const uint32_t v = k < 32 ? m[0] : (k < 64 ? m[1] : (k < 96 ? m[2] : m[3]));
      return (v >> (k & 31)) & 1u;
    }
  };
  // memory row of a sorted position (the position itself without an argsort), -1 past the end
  auto row_of = [&](int pos, int raw) __attribute__((always_inline)) -> int { return pos < p.n_pos ? (has_rows ? raw : pos) : -1; };
  uint32_t key_off = kOob;
  Words key_bits;
  {
    const int pos = key_pos;
    const int row = row_of(pos, raw_key_row);
    const int key = lane < RPW && pos < p.n_pos ? (p.gather_by_pos ? pos : row) : -1;
    key_off = key >= 0 && key < p.n_idx ? (uint32_t)key * 4u : kOob;
    key_bits = row_words(raw_key_bits);
    if (lane >= RPW) key_bits = Words{};
  }
  // ---- tile mask: OR over the tile's positions (cumm/conv/kernel.py:844-889 of the reference)
  uint32_t kmask = 1u;
  uint32_t kwords[MW];         // MW > 1: the tile mask, word by word (kmask is then unused)
#pragma unroll
  for (int w = 0; w < MW; ++w) kwords[w] = w == 0 ? 1u : 0u;
  bool half_skipped = false;   // HALVES: this wave's 64 positions would have been a skipped 64-row tile
  if constexpr (MW > 1) {
    if (has_mask) {
      uint32_t any = 0;
#pragma unroll
      for (int w = 0; w < MW; ++w) {
        kwords[w] = wave_or_dpp(mk[w]) & p.mask_filter;
        any |= kwords[w];
        if (p.mask_out != nullptr && tid == 0 && col == 0 && w < mic && tile * mic + w < p.n_mask_out)
          p.mask_out[tile * mic + w] = kwords[w];
      }
      if (p.exit_on_empty && any == 0) return;
      if (p.reverse_mask) {
        const v4u t = reverse_words(v4u{kwords[0], kwords[MW > 1 ? 1 : 0], kwords[MW > 2 ? 2 : 0], kwords[MW > 3 ? 3 : 0]});
#pragma unroll
        for (int w = 0; w < MW; ++w) kwords[w] = t[w];
      }
#pragma unroll
      for (int w = 0; w < MW; ++w) {
        const int left = p.kv - 32 * w;       // offsets this word may name
        kwords[w] = left >= 32 ? kwords[w] : (left > 0 ? kwords[w] & ((1u << left) - 1u) : 0u);
      }
    }
  } else if (has_mask) {
    kmask = wave_or_dpp(mk[0]) & p.mask_filter;
    if constexpr (HALVES) {
      static_assert(!HALVES || (MKW == 2 && WM == 2), "two mask words of 64 positions, one per row of waves");
      const uint32_t lo = wave_or_dpp((uint32_t)raw_mk[0][0]) & p.mask_filter;
      const uint32_t hi = wave_or_dpp((uint32_t)raw_mk[MKW - 1][0]) & p.mask_filter;
      half_skipped = p.exit_on_empty && (wm == 0 ? lo : hi) == 0u;
      if (p.mask_out != nullptr && tid == 0 && col == 0) {
        if (2 * tile < p.n_mask_out) p.mask_out[2 * tile] = lo;
        if ((2 * tile + 1) * 64 < p.n_pos && 2 * tile + 1 < p.n_mask_out) p.mask_out[2 * tile + 1] = hi;
      }
    } else if constexpr (HALF32) {
      const uint32_t whole = kmask | (wave_or_dpp((uint32_t)raw_other) & p.mask_filter);
      if (p.mask_out != nullptr && tid == 0 && col == 0 && (tile & 1) == 0 && (tile >> 1) < p.n_mask_out) p.mask_out[tile >> 1] = whole;
      if (p.exit_on_empty && whole == 0) return;
    } else {
      if (p.mask_out != nullptr && tid == 0 && col == 0 && tile < p.n_mask_out) p.mask_out[tile] = kmask;
    }
    if (!HALF32 && p.exit_on_empty && kmask == 0) return;
    if (p.reverse_mask) kmask = __builtin_bitreverse32(kmask) >> (32 - p.kv);
    if (p.kv < 32) kmask &= (1u << p.kv) - 1u;
  }
  // a step = one kernel offset x one chunk of the contraction (one chunk unless chunk_shift)
  int n_offsets = __builtin_popcount(kmask);
  if constexpr (MW > 1) {
    n_offsets = 0;
#pragma unroll
    for (int w = 0; w < MW; ++w) n_offsets += __builtin_popcount(kwords[w]);
  }
  const int n_steps = n_offsets << p.chunk_shift;


  const uint32_t g_k_bytes = (uint32_t)p.n_idx * 4u;
  const uint32_t g_bytes = has_gather ? p.gather_bytes : 0u;

  // lane j of klist holds the j-th kernel offset of the tile (-1 past the end): lane b pushes
  // b+1 to the lane of its rank among the set bits, lanes without a bit push into lane 63, which
  // nobody reads; a lane nobody pushed to reads 0.
  // With several mask words the list takes two registers (up to 128 offsets) and every lane works
  // out its own entry: the tile's words are wave-uniform, so lane j picks the word that holds the
  // offset of rank j and finds the position of that set bit by halving.
  constexpr int KL = MW == 1 ? 1 : 2;
  int klist[KL];
  if constexpr (MW == 1) {
    const bool bit = lane < 32 && ((kmask >> lane) & 1u);
    const int rank = __builtin_popcount(kmask & ((1u << (lane & 31)) - 1u));
    klist[0] = __builtin_amdgcn_ds_permute(bit ? rank * 4 : 63 * 4, bit ? lane + 1 : 0) - 1;
  } else {
#pragma unroll
    for (int h = 0; h < KL; ++h) {
      int r = h * 64 + lane;          // rank wanted
      uint32_t m = 0;
      int base = 0;
      bool found = false;
#pragma unroll
      for (int w = 0; w < MW; ++w) {
        const int c = __builtin_popcount(kwords[w]);
        const bool here = !found && r < c;
        m = here ? kwords[w] : m;
        base = here ? 32 * w : base;
        found = found || here;
        r = found ? r : r - c;
      }
      int pos = 0;
#pragma unroll
      for (int width = 16; width >= 1; width >>= 1) {
        const int c = __builtin_popcount(m & ((1u << width) - 1u));
        const bool up = r >= c;
        pos += up ? width : 0;
        r -= up ? c : 0;
        m = up ? m >> width : m;
      }
      klist[h] = found ? base + pos : -1;
    }
  }
  // kernel offset of step j (-1 past the end of the tile's list)
  auto k_of_step = [&](int j) __attribute__((always_inline)) -> int {
    const int i = j >> p.chunk_shift;
    if constexpr (MW == 1) {
      return __builtin_amdgcn_readlane(klist[0], i & 63);
    } else {
      const int lo = __builtin_amdgcn_readlane(klist[0], i & 63);
      const int hi = __builtin_amdgcn_readlane(klist[KL - 1], i & 63);
      return i < 64 ? lo : (i < 128 ? hi : -1);
    }
  };

  auto issue_idx = [&](int j, int *slot) __attribute__((always_inline)) {
    const int k = k_of_step(j);
    const v4i rs = rsrc_words(p.gather, k >= 0 ? g_bytes : 0u);
    dma_b32(rs, lds_addr(slot), has_bit(key_bits, k) ? key_off : kOob, (uint32_t)k * g_k_bytes);
  };
  // The entries of the first offsets are requested now; the address work below (row chunks, weight
  // rows, fragment slots) overlaps their round trip.
  if (n_steps > 0) {
    auto first = [&](auto jc) -> bool {
      issue_idx(decltype(jc)::value, idx_slot(jc));
      return false;
    };
    run_steps(first, std::make_integer_sequence<int, DI>{});
  }

  int a_key[IPA];          // without a pair table the gathered row is the key itself
  uint32_t a_col[IPA];     // byte offset of the fetched chunk inside the gathered row, or kOob
  Words a_bits[IPA];       // mask words of the row
  int a_cpos[IPA];         // first contraction element of the fetched chunk (in the first chunk of the row)
#pragma unroll
  for (int t = 0; t < IPA; ++t) {
    const int r = (wave * IPA + t) * RPI + lrow;
    const int pos = pos_base + r;
    a_bits[t] = row_words(raw_a_bits[t]);
    const int row = row_of(pos, raw_a_row[t]);
    const int key = pos < p.n_pos ? (p.gather_by_pos ? pos : row) : -1;
    a_key[t] = key >= 0 && key < p.n_idx ? key : -1;
    const int c = lchunk ^ swz(r);
    a_cpos[t] = c * PV;
    a_col[t] = a_key[t] >= 0 ? (uint32_t)c * 16u : kOob;
  }
  uint32_t w_voff[IPW];
  int w_cpos[IPW];         // contraction element (WT: contraction row) the lane fetches, first chunk
  // WT: chunk XOR of contraction row e.  A transposing read has, per 16 lanes, four rows e .. e+3
  // and four chunks 4*NBW/8 apart (see wt_rd below), 8 bytes of each.  Rows of 128 bytes (TN = 64)
  // alternate between the halves of the 256 bytes the banks span, so rows e and e+2 must use
  // different chunks: bit 2 follows bit 1 of e.  Rows of 256 bytes (TN = 128) all start at bank 0
  // and the four chunks are two apart: bits 0 and 3 follow bits 0 and 1 of e.
  auto swz_w = [](int e) {
    return LPRW == 8 ? 4 * ((e >> 1) & 1) | 2 * ((e >> 2) & 1) : (e & 1) | 8 * ((e >> 1) & 1) | 2 * ((e >> 2) & 1);
  };
  static_assert(!WT || LPRW == 8 || LPRW == 16, "weight tiles of 64 or 128 channels");
#pragma unroll
  for (int t = 0; t < IPW; ++t) {
    if constexpr (!WT) {
      const int rho = (wave * IPW + t) * RPI + lrow;      // LDS row, fragment order
      const int i = rho & 15, nb = (rho >> 4) % NBW, wq = rho / (16 * NBW);
      const int n = n0 + wq * (16 * NBW) + (i >> 2) * (4 * NBW) + nb * 4 + (i & 3);
      const int c = lchunk ^ swz(rho);
      w_cpos[t] = c * PV;
      w_voff[t] = n < p.k_out ? (uint32_t)((int64_t)n * p.w_stride_n * E::kBytes) + (uint32_t)c * 16u : kOob;
    } else {
      const int e = (wave * IPW + t) * RPIW + lane / LPRW;   // contraction row
      const int c = (lane % LPRW) ^ swz_w(e);                 // chunk of the row this lane fetches
      const int n = n0 + c * PV;
      w_cpos[t] = e;
      w_voff[t] = n < p.k_out ? (uint32_t)(((int64_t)e * p.w_stride_c + n) * E::kBytes) : kOob;
    }
  }

  // ---- reader role: fragment slots (16-byte units) relative to the wave's first row
  int a_rd[KS], w_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int slot = m * LPR + ((s * 4 + q) ^ swz(m));
    a_rd[s] = wm * (RBW * 16) * LPR + slot;
    w_rd[s] = wn * (NBW * 16) * LPR + slot;       // (relative to the weight part)
  }
  // transposing reads: byte address inside the weight part for (k-step s, half h, block nb)
  int wt_rd[WT ? KS : 1][2][WT ? NBW : 1];
  if constexpr (WT) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
          const int e = s * 32 + q * 8 + h * 4 + (m >> 2);
          // first channel (tile local) of the four this address lane points at.  Block nb takes
          // channels 4*nb .. 4*nb+3 of every run of 4*NBW: the lane that holds rows 4q .. 4q+3 of
          // the MFMA result then holds 4*NBW consecutive channels over its blocks (16-byte stores),
          // like the fragment order of the untransposed weights
          const int col = wn * (NBW * 16) + (m & 3) * (4 * NBW) + nb * 4;
          const int chunk = (col / PV) ^ swz_w(e);
          wt_rd[s][h][nb] = e * (LPRW * 16) + chunk * 16 + (col % PV) * E::kBytes;
        }
  }

  // ---- output rows of this lane
  int out_row[RBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int pos = pos_base + (wm * RBW + rb) * 16 + m;
    out_row[rb] = row_of(pos, raw_o_row[rb]);
  }

  // ---- the rows that the epilogue blends in (beta * D) are requested now, as hidden loads that
  // the final wait of the step loop covers: their round trip runs under the loop instead of
  // behind it.  These loads
  // are older than every operand load of the loop, so the counted waits there only get stricter.
  constexpr int CPLW = 4 * NBW;            // consecutive output channels of a lane (not WT)
  constexpr int SRC_W = E::kBytes == 2 ? 4 : CPLW / 4;          // dwords per piece
  constexpr int SRC_N = E::kBytes == 2 ? CPLW / 8 : 1;          // pieces per row
  static_assert(E::kBytes == 1 || CPLW % 8 == 0, "two-byte outputs need NBW >= 2");
  const int ch0 = n0 + wn * (NBW * 16) + q * CPLW;
  auto piece_channel = [&](int i) -> int {
    if constexpr (E::kBytes == 2) return ch0 + i * 8;
    else return ch0;
  };
  typedef int src_vec __attribute__((ext_vector_type(SRC_W)));
  src_vec src_pre[RBW][SRC_N] = {};
  if (p.read_source && !WIDE) {   // (four-byte outputs read their source in the epilogue)
    const v4i rsw_d = rsrc_words(p.D, p.d_bytes);
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb) {
      const int o = out_row[rb];
      const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
      for (int i = 0; i < SRC_N; ++i) {
        const int ch = piece_channel(i);
        const bool ok = row_ok && ch < p.k_out;
        load_hidden_into(src_pre[rb][i], rsw_d, ok ? (uint32_t)((int64_t)o * p.ldd + ch) * (uint32_t)E::kBytes : kOob);
      }
    }
  }

  AccV acc[RBW][NBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) acc[rb][nb] = AccV{0, 0, 0, 0};

  const uint32_t a_row_bytes = (uint32_t)p.lda * E::kBytes;
  const uint32_t w_k_bytes = (uint32_t)p.w_stride_k * E::kBytes;

  // entries of this lane's rows out of the wave's slot (its own loads: no barrier needed)
  auto read_idx = [&](const int *slot, int (&dst)[IPA]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < IPA; ++t) dst[t] = has_gather ? slot[t * RPI + lrow] : a_key[t];
  };
  constexpr int CHUNK_E = LPR * PV;      // contraction elements of a stage row
  auto issue_operands = [&](int j, const int (&src)[IPA], v4i *st, v4i *stw) __attribute__((always_inline)) {
    const int k = k_of_step(j);
    const int cc = j & ((1 << p.chunk_shift) - 1);          // chunk of the contraction
    const int cc_e = cc * CHUNK_E;                           // its first element
    const uint32_t cc_b = (uint32_t)cc * (LPR * 16u);        // ... as bytes inside a row
    const v4i rs_a = rsrc_words(p.A, k >= 0 ? p.a_bytes : 0u);
    const v4i rs_w = rsrc_words(p.W, k >= 0 ? p.w_bytes : 0u);
#pragma unroll
    for (int t = 0; t < IPA; ++t) {
      // a_col is out of range already for a row without a key or a chunk past the contraction;
      // adding a row offset below 2 GiB keeps it out of range
      const uint32_t v = (uint32_t)src[t];
      const uint32_t voff = v < (uint32_t)p.rows_a && has_bit(a_bits[t], k) && cc_e + a_cpos[t] < p.c_in
                                ? v * a_row_bytes + a_col[t] + cc_b
                                : kOob;
      dma_b128(rs_a, lds_addr(st + (wave * IPA + t) * 64), voff, 0u);
    }
    // k = -1 comes with zero records; a transposed weight tile steps CHUNK_E contraction rows
    const uint32_t soff = (uint32_t)k * w_k_bytes + (WT ? (uint32_t)cc_e * (uint32_t)p.w_stride_c * E::kBytes : cc_b);
#pragma unroll
    for (int t = 0; t < IPW; ++t)
      dma_b128(rs_w, lds_addr(stw + (wave * IPW + t) * 64), cc_e + w_cpos[t] < p.c_in ? w_voff[t] : kOob, soff);
  };

  if (n_steps > 0) {
    // ---- prologue (the entries of offsets 0 .. DI-1 are on their way): operands of offsets
    // 0 .. L-1, each followed by the next entries (the order of a step, so the waits count the
    // same everywhere)
    auto fill = [&](auto jc) -> bool {
      constexpr int j = decltype(jc)::value;
      wait_vmcnt<DI - 1 + j * (PER_STEP - 1)>();   // entries of offset j have landed
      int v[IPA];
      read_idx(idx_slot(std::integral_constant<int, j % DI>{}), v);
      issue_operands(j, v, stage(std::integral_constant<int, j % NS>{}), stage_w(std::integral_constant<int, j % NS>{}));
      issue_idx(j + DI, idx_slot(std::integral_constant<int, j % DI>{}));
      return false;
    };
    run_steps(fill, std::make_integer_sequence<int, L>{});

    int done = 0;
    auto step = [&](auto uc) -> bool {
      constexpr int u = decltype(uc)::value;      // step number modulo the ring lengths
      constexpr int sc = u % NS;                  // stage computed in this step
      constexpr int sl = (u + L) % NS;            // stage loaded for offset i + L
      constexpr int si = (u + L) % DI;            // entries of offset i + L, then refilled
      wait_vmcnt<WAIT_OPERANDS>();                // own loads of offset i (and all older ones)
      int v[IPA];
      read_idx(idx_slot(std::integral_constant<int, si>{}), v);   // the barrier hides the LDS round trip
      lds_barrier();
      // fragment reads first: their LDS round trip overlaps the address work of the loads below
      const v4i *st = stage(std::integral_constant<int, sc>{});
      const v4i *stw = stage_w(std::integral_constant<int, sc>{});
      v4i af[RBW][KS], wf[NBW][KS];
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          if constexpr (!WT) {
            wf[nb][s] = stw[w_rd[s] + nb * 16 * LPR];
          } else {
            typedef short v4s __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) v4s *lds_v4s;
            const char *base = reinterpret_cast<const char *>(stw);
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(base + wt_rd[s][0][nb]));
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(base + wt_rd[s][1][nb]));
            typedef short v8s __attribute__((ext_vector_type(8)));
            const v8s both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            wf[nb][s] = __builtin_bit_cast(v4i, both);
          }
        }
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
        for (int s = 0; s < KS; ++s) af[rb][s] = st[a_rd[s] + rb * 16 * LPR];
      issue_operands(done + L, v, stage(std::integral_constant<int, sl>{}), stage_w(std::integral_constant<int, sl>{}));
      issue_idx(done + L + DI, idx_slot(std::integral_constant<int, si>{}));
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
          for (int s = 0; s < KS; ++s) acc[rb][nb] = E::mfma(wf[nb][s], af[rb][s], acc[rb][nb]);
      return ++done >= n_steps;
    };
    constexpr int UNROLL = NS;   // DI == NS: both rings are back at slot 0
    while (!run_steps(step, std::make_integer_sequence<int, UNROLL>{})) {
    }
  }

  wait_vmcnt<0>();   // the loads past the end of the offset list still target this workgroup's LDS
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int i = 0; i < SRC_N; ++i) keep_after_wait(src_pre[rb][i]);
  // (a 64-row tile without any offset is left alone when exit_on_empty is set: so is that half)
  if (HALVES && half_skipped) return;
  // ---- epilogue: lane (q, m) holds, for each of its rows, channels ch0 .. ch0 + 4*NBW - 1.
  // The activation and the blend mode are lifted out of the element loops (one straight-line
  // copy per combination): tested per element they cost more issue slots than the arithmetic.
  const __amdgpu_buffer_rsrc_t rs_c = make_rsrc(p.C, p.c_bytes);
  if constexpr (WIDE) {
    const __amdgpu_buffer_rsrc_t rs_d = make_rsrc(p.D, p.read_source ? p.d_bytes : 0u);
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb) {
      const int o = out_row[rb];
      const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) {
        const int ch = ch0 + nb * 4;
        store_wide_piece(acc[rb][nb], p, rs_c, rs_d, row_ok && ch < p.k_out, o, ch);
      }
    }
    return;
  }
  // MODE: 0 = alpha*acc, 1 = alpha*acc + beta*src, 2 = scale*acc + bias, 3 = ... + beta*src
  auto store_rows = [&](auto act_c, auto mode_c) {
    constexpr int ACT = decltype(act_c)::value;
    constexpr int MODE = decltype(mode_c)::value;
    constexpr bool SRC = (MODE & 1) != 0;
    if constexpr (E::kBytes == 2) {
      constexpr int NG = CPLW / 8;   // 16-byte groups
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        const int o = out_row[rb];
        const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const int ch = ch0 + g * 8;
          const bool ok = row_ok && ch < p.k_out;
          const uint32_t coff = ok ? (uint32_t)((int64_t)o * p.ldc + ch) * 2u : kOob;
          v4i src = {0, 0, 0, 0};
          if constexpr (SRC) src = __builtin_bit_cast(v4i, src_pre[rb][g]);
          const uint16_t *sh = reinterpret_cast<const uint16_t *>(&src);
          v4i outv;
          uint16_t *oh = reinterpret_cast<uint16_t *>(&outv);
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const float a = acc[rb][g * 2 + (x >> 2)][x & 3];
            float t = SRC ? __builtin_fmaf(p.alpha, a, p.beta * E::to_float(sh[x])) : p.alpha * a;
            t = apply_act(t, ACT, p.act_alpha);
            oh[x] = E::from_float(t);
          }
          store_out_b128(outv, rs_c, coff, p.stream_stores != 0);
        }
      }
    } else {
      // one-byte outputs: the lane's 4*NBW consecutive channels are 8 or 16 bytes of the row.
      // Scale and bias of these channels were requested when the kernel started.
      constexpr int ND = CPLW / 4;
      typedef int vNi __attribute__((ext_vector_type(ND)));
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        const int o = out_row[rb];
        const bool ok = o >= 0 && o < p.rows_c && ch0 < p.k_out;
        const uint32_t coff = ok ? (uint32_t)((int64_t)o * p.ldc + ch0) : kOob;
        vNi src = {};
        if constexpr (SRC) src = __builtin_bit_cast(vNi, src_pre[rb][0]);
        const int8_t *sb = reinterpret_cast<const int8_t *>(&src);
        vNi outv;
        int ob[CPLW];
#pragma unroll
        for (int x = 0; x < CPLW; ++x) {
          const int a = acc[rb][x >> 2][x & 3];
          float t;
          if constexpr (MODE >= 2) {
            t = __builtin_fmaf(scale_v[x], (float)a, bias_v[x]);
            if constexpr (SRC) t = __builtin_fmaf(p.beta, (float)sb[x], t);
          } else if constexpr (SRC) {
            t = __builtin_fmaf(p.alpha, (float)a, p.beta * (float)sb[x]);
          } else {
            t = p.alpha * (float)a;
          }
          t = apply_act(t, ACT, p.act_alpha);
          ob[x] = f32_to_s8(t);
        }
#pragma unroll
        for (int g = 0; g < ND; ++g) outv[g] = pack4_bytes(ob[4 * g], ob[4 * g + 1], ob[4 * g + 2], ob[4 * g + 3]);
        if constexpr (ND == 4) store_out_b128(outv, rs_c, coff, p.stream_stores != 0);
        else store_out_b64(outv, rs_c, coff, p.stream_stores != 0);
      }
    }
  };
  auto with_mode = [&](auto act_c) {
    const int mode = (p.read_source ? 1 : 0) | (E::kBytes == 1 && p.int8_epilogue ? 2 : 0);
    switch (mode) {
    case 0: store_rows(act_c, std::integral_constant<int, 0>{}); break;
    case 1: store_rows(act_c, std::integral_constant<int, 1>{}); break;
    case 2: if constexpr (E::kBytes == 1) store_rows(act_c, std::integral_constant<int, 2>{}); break;
    default: if constexpr (E::kBytes == 1) store_rows(act_c, std::integral_constant<int, 3>{}); break;
    }
  };
  switch (p.act) {
  case 1: with_mode(std::integral_constant<int, 1>{}); break;
  case 2: with_mode(std::integral_constant<int, 2>{}); break;
  case 3: with_mode(std::integral_constant<int, 3>{}); break;
  default: with_mode(std::integral_constant<int, 0>{}); break;
  }
}

template <class T, int WM, int WN, int RBW, int NBW, int KS, int NS, bool WT = false, bool WIDE = false, int MW = 1>
__global__ __launch_bounds__(WM *WN * 64) void rowgemm_lds_kernel(const RowGemmParams p) {
  constexpr int NW = WM * WN;
  constexpr int LPR = 4 * KS;
  constexpr int A_V = WM * RBW * 16 * LPR;
  constexpr int STAGE_V = (WM * RBW * 16 + WN * NBW * 16) * LPR;
  __shared__ v4i st0[STAGE_V];
  __shared__ v4i st1[STAGE_V];
  __shared__ v4i st2[NS > 2 ? STAGE_V : 1];
  __shared__ v4i st3[NS > 3 ? STAGE_V : 1];
  // pair-table entries also travel global -> LDS directly: every vector load of the step loop is
  // then counted by hand, none returns into a register the compiler would guard with waits of
  // its own.  Slot [d][wave][l] is written by lane l of the wave (lanes >= RPW write zeros).
  // (one array per slot, like the stages)
  __shared__ int ix0[NW][64];
  __shared__ int ix1[NW][64];
  __shared__ int ix2[NS > 2 ? NW : 1][64];
  __shared__ int ix3[NS > 3 ? NW : 1][64];
  const LdsRing lds = {{st0, st1, st2, st3}, {st0 + A_V, st1 + A_V, NS > 2 ? st2 + A_V : st2, NS > 3 ? st3 + A_V : st3},
                       {ix0, ix1, ix2, ix3}};

  // Workgroups are dispatched in the order of their linear number, round-robin over the 8 XCDs.
  // With several column blocks per row tile, the workgroups of one row tile are given numbers 8
  // apart - neighbours in time on one XCD - so that the rows one of them gathers are in that
  // XCD's L2 for the others (as grid.y they would run a whole grid.x apart).
  int tile_rank = (int)blockIdx.x, col = 0;
  if (gridDim.y > 1) {
    const int gx = (int)gridDim.x, gy = (int)gridDim.y;
    const int lin = (int)blockIdx.y * gx + (int)blockIdx.x;
    const int gx8 = gx & ~7;
    if (lin < gx8 * gy) {
      const int slot = lin >> 3;
      tile_rank = (slot / gy) * 8 + (lin & 7);
      col = slot % gy;
    } else {
      const int rest = lin - gx8 * gy;
      tile_rank = gx8 + rest / gy;
      col = rest % gy;
    }
  }
  const int tile = (int)gridDim.x - 1 - tile_rank;  // heaviest tiles first (masks sorted ascending)
  rowgemm_lds_tile<T, WM, WN, RBW, NBW, KS, NS, WT, WIDE, false, MW>(p, tile, col, lds);
}

// Tiles of two shapes in one launch, for one column block of 64 channels (grid.x = number of
// 64-row tiles): the first p.pair_tiles runs of 128 sorted positions are taken as 128-row tiles
// with a ring of two stages, the rest as 64-row tiles with three.  What it is for: the light end
// of the ascending mask order (a submanifold layer's centre-only masks are the smallest mask
// value and lead it: two thirds of the positions of a LiDAR sweep), where a tile has one or two
// kernel offsets and its life is its three dependent memory round trips, not its bytes, so that
// the launch is bound by how many workgroups it has to turn over.  Both rings fill the same LDS
// (three blocks of 64 rows + 64 weight rows, or two blocks of 128 rows and both weight tiles in
// the third), so the occupancy is that of the 64-row kernel.  Any split gives the same bits; a
// many-offset tile in the 128-row part only runs slower (two stages).  Workgroups are dispatched
// in the order of their number: the 64-row tiles first, heaviest first, then the pairs; the
// numbers left over leave at once, last of all.
// workgroups a mixed launch has beyond one per 64-row tile: for the halves of the heavy end
__host__ __device__ constexpr int mixed_spare_tiles(int tiles) { return tiles / 8; }

template <class T, int KS, bool WT>
__global__ __launch_bounds__(256) void rowgemm_lds_mixed_kernel(const RowGemmParams p) {
  constexpr int R64 = 64 * 4 * KS;        // 16-byte vectors of 64 rows
  __shared__ v4i st0[2 * R64];
  __shared__ v4i st1[2 * R64];
  __shared__ v4i st2[2 * R64];
  __shared__ int ix0[4][64];
  __shared__ int ix1[4][64];
  __shared__ int ix2[4][64];
  const int tiles = (p.n_pos + 63) >> 6;      // = gridDim.x, without waiting for the dispatch packet's own load
  // The slot is read whole and without conditions - one scalar load of 32 bytes, one round trip -
  // and compared without short cuts (a chain of && became a chain of dependent loads, each with
  // its own wait); the host always passes a slot, an all-zero one when there is no table.
  typedef int v8i __attribute__((ext_vector_type(8)));
  const v8i slot = *reinterpret_cast<const v8i *>(p.hint_slot);
  const uint64_t mask_addr = (uint64_t)p.mask;
  // (the two filters have to agree on the bits a mask can have: those of the kernel volume)
  const uint32_t live_bits = p.kv < 32 ? (1u << p.kv) - 1u : ~0u;
  const bool named = (slot[0] == (int)(uint32_t)mask_addr) & (slot[1] == (int)(uint32_t)(mask_addr >> 32)) &
                     (slot[2] == p.n_pos) & ((((uint32_t)slot[3] ^ p.mask_filter) & live_bits) == 0u);
  // (a count from the caller comes with a slot that names nothing: one of the two is zero, and the
  // OR keeps the slot's load out of a branch, where it would wait for the pointer first)
  const int hinted = p.pair_tiles | ((named & (slot[4] > 0)) ? slot[4] >> 7 : 0);
  const int pairs = hinted < (tiles >> 1) ? hinted : (tiles >> 1);
  // The heavy end: the 64-row tiles from slot word 5 on are taken as two halves of 32 rows each,
  // which halves the life of the launch's longest tiles - when they are few (an eighth of the
  // tiles at most: the grid has that many workgroups to spare) and lie behind the pairs.
  // (rows of 64 bytes: a 32-row stage is less than one load instruction per wave - no halves)
  const int heavy_tile = named && KS == 2 ? slot[5] >> 6 : tiles;
  const int heavy = heavy_tile >= 2 * pairs && heavy_tile < tiles && tiles - heavy_tile <= mixed_spare_tiles(tiles) ? tiles - heavy_tile : 0;
  const int halves = 2 * heavy;
  const int singles = tiles - 2 * pairs - heavy;
  const int rank = (int)blockIdx.x;
  // dispatch order: the halves of the heavy end (last positions first), the 64-row tiles, heaviest
  // first, then the pairs; the workgroup numbers left over leave at once, last of all
  if (rank < halves) {
    if constexpr (KS == 2) {
      constexpr int R32 = 32 * 4 * KS;      // 16-byte vectors of 32 rows
      const LdsRing lds = {{st0, st1, st2, nullptr}, {st0 + R32, st1 + R32, st2 + R32, nullptr}, {ix0, ix1, ix2, nullptr}};
      rowgemm_lds_tile<T, 2, 2, 1, 2, KS, 3, WT, false, false, 1, true>(p, 2 * tiles - 1 - rank, 0, lds);
    }
  } else if (rank - halves < singles) {
    const LdsRing lds = {{st0, st1, st2, nullptr}, {st0 + R64, st1 + R64, st2 + R64, nullptr}, {ix0, ix1, ix2, nullptr}};
    rowgemm_lds_tile<T, 2, 2, 2, 2, KS, 3, WT, false, false>(p, tiles - heavy - 1 - (rank - halves), 0, lds);
  } else if (rank - halves - singles < pairs) {
    const LdsRing lds = {{st0, st1, nullptr, nullptr}, {st2, st2 + R64, nullptr, nullptr}, {ix0, ix1, nullptr, nullptr}};
    rowgemm_lds_tile<T, 2, 2, 4, 2, KS, 2, WT, false, true>(p, pairs - 1 - (rank - halves - singles), 0, lds);
  }
}

}  // namespace cummhip
