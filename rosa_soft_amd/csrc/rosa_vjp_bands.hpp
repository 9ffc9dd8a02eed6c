// The diagonal-band kernels of the surrogate backward: row maxima, row statistics and
// gradients, as templates over the tile shape.  rosa_vjp_instances.hip instantiates them,
// one translation unit per tile family, so that the families compile side by side;
// rosa_kernels.hip plans the launches and reaches the kernels through vjp_kernel_table().
#pragma once

#include "rosa_device_common.hpp"

namespace {

struct VjpParams {
  Layout L;
  const uint32_t* packed_query;
  const uint32_t* packed_key;
  const uint32_t* value_bits;   // [value_words_total][NVW], head-major over value heads
  const uint16_t* grad_rows;    // [head-major row][grad_pitch] bfloat16 terms of grad_output
  int grad_terms;               // terms per element: 3 for float32, 2 for float16, 1 for bfloat16
  int grad_pitch;               // elements per row: terms * dvp rounded up to whole 32s
  float4* stats;                // [head-major row] (reference logit, denominator, numerator, base)
  const int64_t* dropout_seed;
  float scale, dropout_p, inverse_keep, mismatch_scale;
  float gate_log2;              // mismatch_scale * log2(e) / D
  float logit_gain;             // scale * (sqrt2+1) * log2(e)
  float null_logit;             // 0.5 * scale
  float tail_threshold;         // window products below this are treated as zero in the reverse sweep
  int gradient_mask;
  int dvp;                      // padded value width
  float* grad_query;            // symbol-space accumulators: the gradient tensors themselves
  float* grad_key;              //   (token-major) or, for rows of at most 8 floats, head-major
  float* grad_value;            //   accumulators in the workspace (see symbols_by_head)
  // Global float atomics cost one operation per 64-byte segment an instruction touches.  A
  // row of at most 8 floats is half a segment, and in a token-major tensor the rows a band
  // completes lie H * D floats apart; in a head-major accumulator [sequence, head][position][D]
  // they are neighbours, so that two rows leave in one segment.  Query rows are stored one
  // position down (row t at t - 1) and value rows likewise (route a at a - 1): the first
  // row of a chunk then starts a segment, and the slot of the last position of every
  // (sequence, head) run stays zero.  finalize_gradients_kernel moves the sums to the tensors.
  int symbols_by_head;          // grad_query / grad_key point to head-major accumulators
  int values_by_head;           // grad_value points to a head-major accumulator
  int32_t* work_counter;
  const int32_t* header;        // [0] offsets flag, [1] work counter, [3] chunk records fit,
                                // [4] the row-statistics pass met a long match
  float* checkpoints;           // one record per (band, 16-row chunk), or NULL
  int record_floats;            // kCheckpointFloats (+ kKeepBitFloats with dropout)
  int value_stride;             // value width of the tensors (L.Dv is the slice being processed)
  int value_offset;             // first value dimension of the slice
  float* block_scratch;         // per resident block: ring + segment checkpoints
  int64_t block_scratch_floats;
  int segment_group;            // segments per group of the fallback checkpoints (see carve_vjp)
  int ring_rows;                // W + 1 clipped to the longest possible diagonal
  int total_units;
  int wave_lds_floats;          // LDS floats each wave of a gradient block owns
  int exchange_tile_floats;     // LDS floats of an accumulator tile passed between waves
  int row_queue;                // row tiles travel from band to band through LDS (two-wave blocks)
  int piece_rows;               // rows of a piece of a band in the gradient pass (0: whole bands)
  int max_pieces;               // work items per band: pieces of the longest possible band
};

// Terms of the bfloat16 expansion of a float: x = t0 + t1 + t2 exactly (each term is the
// bfloat16 nearest to what the terms before it leave), so that products with x can run on
// the bfloat16 matrix pipe without losing float32 accuracy.  A float16 value needs two
// terms, a bfloat16 value one.
__device__ __forceinline__ uint32_t bf16_nearest(float x) {
  // round to nearest even on the upper 16 bits; NaN stays NaN
  const uint32_t bits = __float_as_uint(x);
  if ((bits & 0x7fffffffu) > 0x7f800000u) return (bits >> 16) | 0x40u;
  return (bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16;
}

constexpr int kMaxGradTerms = 3;

__host__ __device__ constexpr int grad_term_pitch(int terms, int dvp) {
  return ((terms * dvp + 31) / 32) * 32;  // bfloat16 elements per row: whole 32-wide k blocks
}

// ---------------------------------------------------------------------------
// backward: diagonal-band sweeps
// ---------------------------------------------------------------------------

template <int NVW>
struct Band {
  // sliding per-column registers (lane l holds the column a = a0 - l)
  uint32_t key_word;      // key word of column a     (key position a - 1)
  uint32_t old_key_word;  // key word of column a - W - 1, leaving the window
  // per-diagonal state
  float evidence;   // S of the previous row on this diagonal
  int window;       // mismatching bits over the last min(n, W + 1) gates
};

struct BandView {
  const uint32_t* q;       // head-major words of this (sequence, head)
  const uint32_t* k;
  const uint32_t* vbits;   // value sign words of this (sequence, value head), NVW per token
  const uint16_t* grad_rows;  // [t][grad_pitch] bfloat16 terms
  float4* stats;           // [t]
  float* checkpoints;      // chunk records of this band, or NULL
  int record_floats;
  int len;
  int diag0;               // first diagonal of the band
  int steps;               // rows of the band: t = diag0 + 1 + i
};

// Load the sliding registers so that the shift of step i produces columns a0 - l, a0 = i + 1.
template <int NVW>
__device__ __forceinline__ void load_sliding(Band<NVW>& band, const BandView& view, int i,
                                             int lane, int W) {
  const int a = i - lane;  // column held before the shift
  band.key_word = (a >= 1) ? view.k[a - 1] : 0u;
  band.old_key_word = (a - W - 2 >= 0) ? view.k[a - W - 2] : 0u;
}

// Everything a step needs that depends on the row only is staged in LDS for a
// whole block of rows with one coalesced round trip (lane = row), so that the
// recurrences themselves never wait on memory: a step reads its row with
// wave-uniform LDS loads.  Staged words per row:
//   0 query word of row t          1 query word of row t - W - 1
//   2 key word entering at lane 0  3 key word of column a0 - W - 1 entering at lane 0
//   4 exponent shift of the row    5 expected dropped utility
//   6,7 unused
// In the row-statistics pass the shift is that of the raw weight; in the gradient
// pass the row records are final and the shift includes log2 of the denominator,
// so that exp2 gives the route probability directly.
constexpr int kRowWords = 8;
enum RowDetail { kRowSymbols = 0, kRowStats = 1, kRowFull = 2 };

template <int NVW, int DETAIL>
__device__ __forceinline__ void stage_rows(const BandView& view, int first, int count, int lane,
                                           uint32_t* rows, int W) {
  for (int index = lane; index < count; index += kWave) {
    const int i = min(first + index, view.steps - 1);  // rows past the band's end repeat the last
    const int t = view.diag0 + 1 + i;
    const int a0 = i + 1;
    uint4 symbols;
    symbols.x = view.q[t];
    symbols.y = (t - W - 1 >= 0) ? view.q[t - W - 1] : 0u;
    symbols.z = view.k[a0 - 1];
    symbols.w = (a0 - W - 2 >= 0) ? view.k[a0 - W - 2] : 0u;
    uint4* dst = reinterpret_cast<uint4*>(rows + index * kRowWords);
    dst[0] = symbols;
    if constexpr (DETAIL == kRowStats) {
      const float4 row = view.stats[t];
      dst[1] = make_uint4(__float_as_uint(fmaf(row.x, kLog2e, row.w)), 0u, 0u, 0u);
    } else if constexpr (DETAIL == kRowFull) {
      const uint4 record = reinterpret_cast<const uint4*>(view.stats)[t];  // finalised
      // the replay order of the gradient pass (staged_symbols_replay_order)
      dst[0] = make_uint4(symbols.x, symbols.z, record.y, record.z);
      dst[1] = make_uint4(symbols.y, symbols.w, 0u, 0u);
    }
  }
}

// Value sign words of the window columns of a block of rows: entry `index`
// holds column a = first - 63 + index (zero outside 1 .. len-1).
template <int NVW>
__device__ __forceinline__ void stage_value_columns(const BandView& view, int first, int count,
                                                    int lane, uint32_t* dst) {
  for (int index = lane; index < count * NVW; index += kWave) {
    const int column = index / NVW;
    const int a = first - 63 + column;
    dst[index] = (a >= 1 && a <= view.len - 1)
        ? view.vbits[static_cast<int64_t>(a) * NVW + (index - column * NVW)] : 0u;
  }
}

// bfloat16 terms of the grad_output rows of a block, zero for rows past the band's end;
// `pitch` elements per row in LDS, `source_pitch` in the workspace
__device__ __forceinline__ void stage_grad_rows(const BandView& view, int first, int count,
                                                int lane, uint16_t* dst, int pitch,
                                                int source_pitch) {
  const int pieces = source_pitch / 8;  // 16 bytes each
  for (int index = lane; index < count * pieces; index += kWave) {
    const int r = index / pieces;
    const int piece = index - r * pieces;
    const int i = first + r;
    uint4 value = make_uint4(0u, 0u, 0u, 0u);
    if (i < view.steps) {
      const int t = view.diag0 + 1 + i;
      value = *reinterpret_cast<const uint4*>(view.grad_rows +
                                              static_cast<int64_t>(t) * source_pitch + 8 * piece);
    }
    *reinterpret_cast<uint4*>(dst + r * pitch + 8 * piece) = value;
  }
}

struct StepOut {
  float gate;     // local match gate of this pair
  float overflow; // product of the W+1 gates ending here (0 while the window is not full)
  float evidence; // S(t, a)
  bool active;    // a >= 1
  int a;
};

// the four symbol words a step needs, all wave-uniform
struct RowSymbols {
  uint32_t query;      // q[t]
  uint32_t old_query;  // q[t - W - 1]
  uint32_t key;        // key word of column a0 = i + 1, entering at lane 0
  uint32_t old_key;    // key word of column a0 - W - 1, entering at lane 0
};

__device__ __forceinline__ RowSymbols staged_symbols(const uint32_t* row) {
  const uint4 words = *reinterpret_cast<const uint4*>(row);
  return RowSymbols{words.x, words.y, words.z, words.w};
}

// exp2(-c n) of a mismatch count n without the int -> float conversion: 0x3f800000 + n is
// the float 1 + n 2^-23, and fma(that, -c 2^23, c 2^23) is -c n with the single rounding
// of the plain product.
constexpr int kCountBias = 0x3f800000;

// popcount(x) + kCountBias: the bias is the inline constant 1.0 of the instruction
__device__ __forceinline__ int biased_popc(uint32_t x) {
  int result;
  asm("v_bcnt_u32_b32 %0, %1, 1.0" : "=v"(result) : "v"(x));
  return result;
}

__device__ __forceinline__ float decay_of_biased_count(int biased, float gate_log2) {
  const float slope = gate_log2 * 8388608.0f;
  return fast_exp2(fmaf(__int_as_float(biased), -slope, slope));
}

// One forward step of the evidence recurrence S = g (1 + S_prev) - overflow.
// STEADY: every lane of the wave is past its diagonal's first W + 1 rows, so no
// lane needs masking (true for all but the first W + 64 rows of a band).
// QUIET (with STEADY): the caller knows that no overflow term of these rows can move
// a float32 result; the window is not tracked and the overflow is taken as zero.
// BIASED: Band::window carries kCountBias on top of the count (the caller adds it when
// the band starts and removes it where the count leaves the kernel).
template <int NVW, bool STEADY = false, bool QUIET = false, bool BIASED = false>
__device__ __forceinline__ StepOut forward_step(Band<NVW>& band, const RowSymbols& symbols, int i,
                                                int lane, int W, float gate_log2) {
  const int a0 = i + 1;
  band.key_word = dpp_wave_shr1(symbols.key, band.key_word);
  StepOut out;
  out.a = a0 - lane;
  if constexpr (STEADY && QUIET) {
    out.active = true;
    out.gate = decay_of_biased_count(biased_popc(symbols.query ^ band.key_word), gate_log2);
    out.overflow = 0.0f;
    band.evidence = fmaf(out.gate, band.evidence, out.gate);
    out.evidence = band.evidence;
    return out;
  }
  const int mismatches = __popc(symbols.query ^ band.key_word);
  const auto window_decay = [&]() {
    return BIASED ? decay_of_biased_count(band.window, gate_log2)
                  : fast_exp2(-gate_log2 * static_cast<float>(band.window));
  };
  const float gate = BIASED ? decay_of_biased_count(mismatches + kCountBias, gate_log2)
                            : fast_exp2(-gate_log2 * static_cast<float>(mismatches));
  band.old_key_word = dpp_wave_shr1(symbols.old_key, band.old_key_word);
  if constexpr (STEADY) {
    out.active = true;
    band.window += mismatches - __popc(symbols.old_query ^ band.old_key_word);
    out.gate = gate;
    out.overflow = window_decay();
    band.evidence = fmaf(out.gate, band.evidence, out.gate) - out.overflow;
  } else {
    out.active = out.a >= 1;
    const int leaving = (out.a >= W + 2) ? __popc(symbols.old_query ^ band.old_key_word) : 0;
    band.window =
        out.active ? band.window + mismatches - leaving : (BIASED ? kCountBias : 0);
    out.gate = out.active ? gate : 0.0f;
    out.overflow = (out.a >= W + 1) ? window_decay() : 0.0f;
    const float next = fmaf(out.gate, band.evidence, out.gate) - out.overflow;
    band.evidence = out.active ? next : 0.0f;
  }
  out.evidence = band.evidence;
  return out;
}

// The gradient pass keeps what every row of its replay reads in the first four words:
//   0 query word of row t          1 key word entering at lane 0
//   2 exponent shift of the row    3 expected dropped utility
//   4 query word of row t - W - 1  5 key word of column a0 - W - 1 entering at lane 0
__device__ __forceinline__ RowSymbols staged_symbols_replay_order(const uint32_t* row) {
  const uint2 front = *reinterpret_cast<const uint2*>(row);
  const uint2 back = *reinterpret_cast<const uint2*>(row + 4);
  return RowSymbols{front.x, back.x, front.y, back.y};
}

// Evidence-only sweep over `count` staged rows starting at step `first`.
template <int NVW, bool REPLAY_ORDER = false>
__device__ __forceinline__ void sweep_rows(Band<NVW>& band, const uint32_t* rows, int first,
                                           int count, int lane, int W, float gate_log2) {
  const auto symbols_of = [&](int r) {
    return REPLAY_ORDER ? staged_symbols_replay_order(rows + r * kRowWords)
                        : staged_symbols(rows + r * kRowWords);
  };
  if (first >= W + kWave) {  // steady state: all 64 lanes are past their window fill
#pragma unroll 4
    for (int r = 0; r < count; ++r) {
      forward_step<NVW, true>(band, symbols_of(r), first + r, lane, W, gate_log2);
    }
  } else {
#pragma unroll 4
    for (int r = 0; r < count; ++r) {
      forward_step<NVW, false>(band, symbols_of(r), first + r, lane, W, gate_log2);
    }
  }
}

typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4f mfma_16x16x4(float a, float b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// +1.0f where bit 31 of `x` is clear, -1.0f where it is set
__device__ __forceinline__ float sign_from_bit31(uint32_t x) {
  return __uint_as_float((x & 0x80000000u) | 0x3f800000u);
}

// The contractions run on the bfloat16 matrix pipe: v_mfma_f32_16x16x32_bf16 multiplies a
// 16 x 32 by a 32 x 16 matrix in the time v_mfma_f32_16x16x4_f32 takes for a 16 x 4 by
// 4 x 16 one, with float32 accumulation.  Lane (li, lg) = (lane & 15, lane >> 4) supplies
// row li of A and column li of B for k = 8 lg .. 8 lg + 7 (element 2 j of the operand is the
// low half of its dword j) and receives rows 4 lg .. 4 lg + 3 of column li of the product.
// One factor of every product here is exactly representable (signs, or grad_output as a
// sum of bfloat16 terms); the other one is split into a leading bfloat16 and the bfloat16
// nearest to the rest, which keeps 16 to 17 significant bits of it.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4f mfma_bf16(v4u a, v4u b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a),
                                                 __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}

// [leading | rest << 16] of a float: the bfloat16 nearest to it and the bfloat16 nearest to
// what that leaves.  Adjacent k indices of a matrix operand, so that a product with an
// operand that repeats its element for both gives x (to 2^-17) times that element.
__device__ __forceinline__ uint32_t split_bf16(float x) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  // leading term rounded half up on the upper 16 bits (its conversion below is exact), the
  // rest rounded by the conversion: |x - pair| <= 2^-9 * 2^-8 |x|, without a bias
  const float head = __uint_as_float((__float_as_uint(x) + 0x8000u) & 0xffff0000u);
  const v2f parts = {head, x - head};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(parts, v2bf));
}

// Three-term split of a float by truncation: x = leading + middle + rest to 2^-21 of |x|
// (each term takes the upper 16 bits of what the terms before it leave; the subtractions
// are exact).  Returns [leading | middle << 16]; `rest` receives the third term in the
// upper half of its bits.  (Rounding the third term instead changed no measured error: the
// gate adjoints' own float32 recurrence is what limits dQ and dK.)
__device__ __forceinline__ uint32_t split_bf16_exact(float x, uint32_t& rest) {
  const uint32_t leading = __float_as_uint(x) & 0xffff0000u;
  const float after_leading = x - __uint_as_float(leading);
  const uint32_t middle = __float_as_uint(after_leading) & 0xffff0000u;
  rest = __float_as_uint(after_leading - __uint_as_float(middle));
  return __builtin_amdgcn_perm(middle, leading, 0x07060302u);  // leading >> 16 | middle
}

// 16 x 16 x 16 bfloat16 product: lane (li, lg) supplies k = 4 lg .. 4 lg + 3 (two dwords)
typedef short v4s __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ v4f mfma_bf16_k16(v2u a, v2u b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4s, a),
                                                   __builtin_bit_cast(v4s, b), c, 0, 0, 0);
}

// Between matrix instructions of different shapes that share an accumulator: keeps the
// groups apart for the scheduler and spends the wait states of the longest pipeline.
__device__ __forceinline__ void mfma_shape_change() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// two 16-bit LDS words as one dword: first | second << 16
__device__ __forceinline__ uint32_t pair_of(const uint16_t* first, const uint16_t* second) {
  typedef uint16_t v2h __attribute__((ext_vector_type(2)));
  const v2h both = {*first, *second};
  return __builtin_bit_cast(uint32_t, both);
}

// bfloat16 -1.0 in both halves where bit `bit` of `word` is set, +1.0 where it is clear: the
// negated symbol for both terms of a split operand; callers fold the sign into their scale.
__device__ __forceinline__ uint32_t negated_symbol_pair(uint32_t word, int bit) {
  const int spread = __builtin_amdgcn_sbfe(static_cast<int>(word), bit, 1);  // 0 or all ones
  // (a & b) | c is one instruction when no operand is a literal: the two constants are held
  // in registers, one scalar and one vector (the instruction reads one scalar at most)
  uint32_t sign_bits = 0x80008000u, ones = 0x3f803f80u;
  asm("" : "+s"(sign_bits));
  asm("" : "+v"(ones));
  return (static_cast<uint32_t>(spread) & sign_bits) | ones;
}

// Four sign bits -> four bfloat16 values (+1.0 where the bit is set, -1.0 where it is
// clear) as two dwords: a table of 16 entries, 128 bytes, one entry per LDS bank pair, so
// that any mix of entries is read without a bank conflict.
constexpr int kSignTableWords = 32;

__device__ __forceinline__ void fill_sign_table(uint32_t* table, int lane) {
  if (lane < kSignTableWords) {
    const int nibble = lane >> 1;
    const int low = (nibble >> (2 * (lane & 1))) & 1;
    const int high = (nibble >> (2 * (lane & 1) + 1)) & 1;
    table[lane] = (low ? 0x3f80u : 0xbf80u) | ((high ? 0x3f80u : 0xbf80u) << 16);
  }
}

// Utilities u(t, a) = sum_d grad_output[t, d] * sign(v[a, d]) of 16 rows against
// their 80 window columns on the matrix cores, written in (row r, lane l)
// coordinates: out[r * pitch + l] for the pair on diagonal lane l, whose window
// column is c = 64 - l + r (BY_COLUMN: out[r * pitch + c], pitch a multiple of 4).
// `grad_tile` holds the bfloat16 terms of the 16 grad_output rows, `grad_pitch` elements
// each: k = term * DVP + d, `k_blocks` blocks of 32 (zero beyond the last term); the sum
// over the terms is the float32 product.  `value_columns` holds the sign words of the
// window columns (NVW per column).  Elements of the first and last column tile that
// belong to no lane go to `discard` (one float per lane).
// The five column tiles are taken through each stage together (sign words, table entries,
// matrix products, stores): the LDS and matrix latencies of one tile are covered by the
// others instead of adding up (one tile after the other took 13 % of the gradient kernel,
// together 7 %), at the price of twenty more live registers.
template <int NVW, int DVP, bool BY_COLUMN, int BATCH = 5>
__device__ __forceinline__ void utility_tiles_staged(const uint16_t* grad_tile, int grad_pitch,
                                                     int k_blocks, const uint32_t* value_columns,
                                                     const uint32_t* sign_table, float* out,
                                                     int pitch, float* discard, int lane) {
  const int li = lane & 15;
  const int lg = lane >> 4;
  const uint16_t* a_row = grad_tile + li * grad_pitch + 8 * lg;
  constexpr int kBlocksMax = grad_term_pitch(kMaxGradTerms, DVP) / 32;
  // BATCH tiles at a time (all five where the registers are there)
#pragma unroll
  for (int m0 = 0; m0 < 5; m0 += BATCH) {
    constexpr int kTilesMax = BATCH;
    const int tiles = 5 - m0 < BATCH ? 5 - m0 : BATCH;  // folds: m0 is an unrolled constant
    // (two arrays, not one indexed by the word: a select between elements of one array
    // becomes a dynamic index, and the array then lives in scratch memory)
    uint32_t low_words[kTilesMax], high_words[kTilesMax];
#pragma unroll
    for (int n = 0; n < kTilesMax; ++n) {
      if (n >= tiles) break;
      const int m = m0 + n;
      low_words[n] = value_columns[(16 * m + li) * NVW];
      high_words[n] = NVW > 1 ? value_columns[(16 * m + li) * NVW + NVW - 1] : 0u;
    }
    v4f acc[kTilesMax];
#pragma unroll
    for (int n = 0; n < kTilesMax; ++n) acc[n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int q = 0; q < kBlocksMax; ++q) {
      if (q > 0 && q >= k_blocks) break;  // wave-uniform; there is always a first block
      const v4u a = *reinterpret_cast<const v4u*>(a_row + 32 * q);
      const int d0 = (32 * q + 8 * lg) & (DVP - 1);
      v4u signs[kTilesMax];
#pragma unroll
      for (int n = 0; n < kTilesMax; ++n) {
        if (n >= tiles) break;
        uint32_t word = low_words[n];
        if constexpr (NVW > 1) word = d0 >= 32 ? high_words[n] : low_words[n];
        const uint32_t byte = word >> (d0 & 31);
        const uint2 low = *reinterpret_cast<const uint2*>(sign_table + ((byte << 1) & 0x1e));
        const uint2 high = *reinterpret_cast<const uint2*>(sign_table + ((byte >> 3) & 0x1e));
        signs[n] = v4u{low.x, low.y, high.x, high.y};
      }
#pragma unroll
      for (int n = 0; n < kTilesMax; ++n) {
        if (n >= tiles) break;
        acc[n] = BY_COLUMN ? mfma_bf16(signs[n], a, acc[n]) : mfma_bf16(a, signs[n], acc[n]);
      }
    }
    // The products are read right behind a branch of the loop above, where the compiler has
    // been seen to leave out the wait states a matrix result needs before vector or LDS
    // instructions may read it (wrong utilities): they are spent here, once for the batch.
    if constexpr (BATCH == 5) {
      asm volatile("s_nop 7\n\ts_nop 3"
                   : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]));
    } else {
#pragma unroll
      for (int n = 0; n < kTilesMax; ++n) asm volatile("s_nop 7\n\ts_nop 3" : "+v"(acc[n]));
    }
#pragma unroll
    for (int n = 0; n < kTilesMax; ++n) {
      if (n >= tiles) break;
      const int m = m0 + n;
      if constexpr (BY_COLUMN) {
        const int r = li;
        const int c = 16 * m + 4 * lg;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (m == 0 && c + e < r + 1) acc[n][e] = 0.0f;
          if (m == 4 && c + e > r + kWave) acc[n][e] = 0.0f;
        }
        *reinterpret_cast<v4f*>(out + r * pitch + c) = acc[n];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * lg + e;
          const int l = 64 - (16 * m + li) + r;
          float* target = out + r * pitch + l;
          if (m == 0) target = l < kWave ? target : discard + lane;
          if (m == 4) target = l >= 0 ? target : discard + lane;
          *target = acc[n][e];
        }
      }
    }
  }
}

template <int NVW, bool VARLEN>
__device__ __forceinline__ bool make_view(const VjpParams& P, const Unit& u, BandView& view,
                                          int& value_head) {
  view.len = u.len;
  view.diag0 = u.block * kWave;
  view.steps = u.len - 1 - view.diag0;
  if (view.steps <= 0) return false;
  view.q = P.packed_query + u.word_base;
  view.k = P.packed_key + u.word_base;
  value_head = u.head / (P.L.H / P.L.Hv);
  const int64_t value_base = VARLEN
      ? static_cast<int64_t>(value_head) * P.L.N + u.start
      : (static_cast<int64_t>(u.seq) * P.L.Hv + value_head) * P.L.T;
  view.vbits = P.value_bits + value_base * NVW;
  view.grad_rows = P.grad_rows + u.word_base * P.grad_pitch;
  view.stats = P.stats + u.word_base;
  // position of the band in the global (step, band) order of the cached data
  int64_t steps_before, bands_before;
  const int blocks = (u.len + 63) >> 6;
  if constexpr (VARLEN) {
    steps_before = P.L.step_prefix[u.seq] * P.L.H + u.head * band_steps_total(u.len);
    bands_before = static_cast<int64_t>(P.L.block_prefix[u.seq]) * P.L.H + u.head * blocks;
  } else {
    const int64_t sequence_head = static_cast<int64_t>(u.seq) * P.L.H + u.head;
    steps_before = sequence_head * band_steps_total(u.len);
    bands_before = sequence_head * blocks;
  }
  steps_before += band_steps_before(u.len, u.block);
  bands_before += u.block;
  view.checkpoints = nullptr;
  view.record_floats = P.record_floats;
  if (P.checkpoints != nullptr && (!VARLEN || P.header[3] != 0)) {
    view.checkpoints = P.checkpoints + ((steps_before >> 4) + bands_before) * P.record_floats;
  }
  return true;
}

// Row-maximum pass (only when the analytic bound is too loose to be a safe
// exponent reference): raises stats[t].x to the largest logit of the row.
template <int NVW, bool VARLEN>
__global__ __launch_bounds__(kWave) void vjp_row_max_kernel(VjpParams P) {
  __shared__ __attribute__((aligned(16))) uint32_t rows[kWave * kRowWords];
  const Unit u = decode_unit<VARLEN>(P.L, blockIdx.x);
  if (!u.valid) return;
  BandView view;
  int hv;
  if (!make_view<NVW, VARLEN>(P, u, view, hv)) return;
  const int lane = threadIdx.x;
  const int W = P.L.W;
  Band<NVW> band;
  band.evidence = 0.0f;
  band.window = 0;
  load_sliding<NVW>(band, view, 0, lane, W);
  for (int first = 0; first < view.steps; first += kWave) {
    const int count = min(kWave, view.steps - first);
    wave_lds_fence();
    stage_rows<NVW, kRowSymbols>(view, first, count, lane, rows, W);
    wave_lds_fence();
    for (int r = 0; r < count; ++r) {
      const int i = first + r;
      const StepOut s =
          forward_step<NVW>(band, staged_symbols(rows + r * kRowWords), i, lane, W, P.gate_log2);
      const int t = view.diag0 + 1 + i;
      const float root = sqrtf(1.0f + s.evidence);
      const float logit = P.scale * kSqrtScale * (root - 1.0f) - logf(static_cast<float>(t));
      float best = s.active ? fmaxf(logit, 0.0f) : 0.0f;
      best = wave_max_lane63(best);
      if (lane == 63) {
        atomicMax(reinterpret_cast<int*>(&view.stats[t].x), __float_as_int(best));
      }
    }
  }
}

// 2 * bits + (flag ? 1 : 0) as one add with carry (the compiler builds a select, a shift and
// an or from the plain expression).
__device__ __forceinline__ uint32_t doubled_plus_flag(uint32_t bits, bool flag) {
  const uint64_t carry_in = __builtin_amdgcn_ballot_w64(flag);
  uint64_t carry_out;
  uint32_t result;
  asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3"
      : "=v"(result), "=s"(carry_out)
      : "v"(bits), "s"(carry_in));
  return result;
}

// Sum of every row of a [16][pitch] LDS tile over its 64 columns: each lane adds four
// neighbouring columns (one 16-byte read), and the matrix cores add the 16 partial sums
// of a row (the partial sums times a matrix of ones).  `pitch` is a multiple of 4 floats.
// Lane (li, lg) = (lane & 15, lane >> 4) returns with the sums of rows 4 lg + e in
// element e, whatever li.
template <int ROWS>
__device__ __forceinline__ v4f tile_row_sums(const float* tile_rows, int pitch, int lane) {
  const int li = lane & (ROWS - 1);  // a tile of eight rows repeats in the product
  const int lg = lane >> 4;
  // a lane adds its 16 columns (four aligned 16-byte words of row li) and one product with a
  // matrix of ones adds the four lanes of a row: float32 matrix instructions keep the
  // vector pipe of the SIMD waiting, so there is one per tile, not one per word
  float partial = 0.0f;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const float4 part =
        *reinterpret_cast<const float4*>(tile_rows + li * pitch + 16 * ks + 4 * lg);
    partial += (part.x + part.y) + (part.z + part.w);
  }
  return mfma_16x16x4(partial, 1.0f, v4f{0.0f, 0.0f, 0.0f, 0.0f});
}

// Waves per SIMD the row-statistics kernel is compiled for (no variant spills at these; the
// widest tile with dropout is one register short of four).  Its LDS allows four with 16-bit
// inputs at every width.
constexpr int row_stats_waves(int dvp, bool dropout) { return dvp > 32 && dropout ? 3 : 4; }

constexpr float kLongMatchEvidence = 6.0f;

// Row-statistics pass: denominator and expected dropped utility of every row.
// Rows are processed 16 at a time without any branch in between.  A chunk leaves
// its route weights and its dropped weighted utilities as two [row][lane] tiles
// in LDS; their row sums are formed on the matrix cores and leave in one atomic
// each from 16 lanes; every lane keeps its 16 dropout decisions of the chunk as bits and
// stores them with the chunk's checkpoint for the gradient pass.
template <int NVW, int DVP, bool VARLEN, bool DROPOUT>
__global__ __launch_bounds__(kWave)
__attribute__((amdgpu_waves_per_eu(row_stats_waves(DVP, DROPOUT))))
void vjp_row_stats_kernel(VjpParams P) {
  // rows staged in LDS at a time: one chunk, loaded a chunk ahead.  With the half-height
  // weight tile below a block's LDS stays under 10 KB, which lets four waves share a SIMD
  constexpr int kBlockRows = kChunk;
  constexpr int kUtilityPitch = 68;  // rows 16-byte aligned, 16 lanes of a row read 64 banks
  constexpr int kWeightPitch = 68;
  __shared__ __attribute__((aligned(16))) uint32_t rows[kBlockRows * kRowWords];
  // bfloat16 terms of the block's grad_output rows, 16 bytes of padding per row against
  // bank conflicts of the operand reads; sized at the launch for the terms the input type
  // needs (row_stats_dynamic_lds), because the LDS of a block bounds the waves per SIMD
  constexpr int kGradChunksMax = grad_term_pitch(kMaxGradTerms, DVP) / 8;  // 16-byte pieces per row
  extern __shared__ __attribute__((aligned(16))) uint16_t grads[];  // [kBlockRows][grad_pitch + 8]
  __shared__ __attribute__((aligned(16))) uint32_t sign_table[kSignTableWords];
  __shared__ uint32_t value_columns[(kBlockRows + kWave) * NVW];
  __shared__ __attribute__((aligned(16))) float utilities[kChunk * kUtilityPitch];  // u, then e d u
  // e, eight rows at a time (their sums are taken after rows 7 and 15); while the utilities
  // are formed it takes the elements of the edge tiles that belong to no lane
  constexpr int kWeightRows = kChunk / 2;
  __shared__ __attribute__((aligned(16))) float weights[kWeightRows * kWeightPitch];
  float* const discard = weights;
  const Unit u = decode_unit<VARLEN>(P.L, blockIdx.x);
  if (!u.valid) return;
  BandView view;
  int hv;
  if (!make_view<NVW, VARLEN>(P, u, view, hv)) return;
  const int lane = threadIdx.x;
  const int W = P.L.W;
  DropoutKey key;
  if constexpr (DROPOUT) {
    key = make_dropout_key(static_cast<uint64_t>(*P.dropout_seed), u.head, u.seq, P.dropout_p);
    // the keys of the rounds that every pair runs: one xor each, at the rate of simple
    // instructions only with vector operands
    key.head_key = in_vector_register(key.head_key);
    key.batch_key = in_vector_register(key.batch_key);
    key.seed_low_key = in_vector_register(key.seed_low_key);
    key.seed_high_key = in_vector_register(key.seed_high_key);
  }
  const float logit_gain = in_vector_register(P.logit_gain);
  Band<NVW> band;
  band.evidence = 0.0f;
  band.window = kCountBias;  // forward_step<..., BIASED>
  load_sliding<NVW>(band, view, 0, lane, W);
  const bool needs_utility = (P.gradient_mask & (ROSA_GRAD_QUERY | ROSA_GRAD_KEY)) != 0;
  uint32_t route_hash = route_hash_of(-lane);
  const int last_step = view.steps - 1;
  // without symbol gradients no utilities are computed and the tile stays zero
  for (int index = lane; index < kChunk * kUtilityPitch; index += kWave) utilities[index] = 0.0f;
  fill_sign_table(sign_table, lane);
  // windows with at least this many mismatching bits at the start of a chunk stay above the
  // count whose overflow term exp2(-gate_log2 * count) reaches tail_threshold
  const int quiet_window =
      static_cast<int>(ceilf(-__log2f(P.tail_threshold) / P.gate_log2)) + kChunk * P.L.D + 1;
  const int grad_chunks = P.grad_pitch / 8;   // 16-byte pieces per row actually present
  const int grad_lds_pitch = P.grad_pitch + 8;
  // The global loads of a block (row words, row records, grad_output pieces, value sign
  // words) set out one block ahead, into registers, right after the block before has been
  // stored to LDS: a memory round trip per 32 rows was a fifth of a wave's time.  The
  // grad_output rows come as 16-byte pieces, numbered row by row over the pieces the input
  // type really has, in groups of at most two registers per lane: the first group travels
  // ahead with the other loads, later ones (float32 rows of wider tiles) take a round trip of
  // their own when the block starts instead of the registers the chunk loop needs.
  constexpr int kGradParts = (kBlockRows * kGradChunksMax + kWave - 1) / kWave;
  constexpr int kGradGroup = kGradParts < 2 ? kGradParts : 2;
  constexpr int kValueParts = ((kBlockRows + kWave) * NVW + kWave - 1) / kWave;
  const int pieces = kBlockRows * grad_chunks;
  const float per_row = 1.0f / static_cast<float>(grad_chunks);
  uint4 symbols_in;
  float4 stat_in;
  uint4 grad_in[kGradGroup];
  uint32_t value_in[kValueParts];
  const auto load_pieces = [&](int first, int group) {
    // (the piece numbering is recomputed where it is used: kept across the chunk loop it
    // would cost registers the wider variants do not have)
    int piece_lane = lane;
    asm volatile("" : "+v"(piece_lane));
#pragma unroll
    for (int part = 0; part < kGradGroup; ++part) {
      const int index = (group + part) * kWave + piece_lane;
      const int r = static_cast<int>((static_cast<float>(index) + 0.5f) * per_row);
      const int piece = index - r * grad_chunks;
      grad_in[part] = make_uint4(0u, 0u, 0u, 0u);
      if (index < pieces && first + r < view.steps) {
        grad_in[part] = *reinterpret_cast<const uint4*>(
            view.grad_rows + static_cast<int64_t>(view.diag0 + 1 + first + r) * P.grad_pitch +
            8 * piece);
      }
    }
  };
  const auto store_pieces = [&](int group) {
    int piece_lane = lane;
    asm volatile("" : "+v"(piece_lane));
#pragma unroll
    for (int part = 0; part < kGradGroup; ++part) {
      const int index = (group + part) * kWave + piece_lane;
      const int r = static_cast<int>((static_cast<float>(index) + 0.5f) * per_row);
      const int piece = index - r * grad_chunks;
      if (index < pieces) {
        *reinterpret_cast<uint4*>(grads + r * grad_lds_pitch + 8 * piece) = grad_in[part];
      }
    }
  };
  const auto issue_block_loads = [&](int first) {
    const int i = min(first + lane, view.steps - 1);  // rows past the band's end repeat the last
    const int t = view.diag0 + 1 + i;
    symbols_in = make_uint4(0u, 0u, 0u, 0u);
    stat_in = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (lane < kBlockRows) {
      symbols_in.x = view.q[t];
      symbols_in.y = (t - W - 1 >= 0) ? view.q[t - W - 1] : 0u;
      symbols_in.z = view.k[i];
      symbols_in.w = (i - W - 1 >= 0) ? view.k[i - W - 1] : 0u;
      stat_in = view.stats[t];
    }
    if (needs_utility) {
      load_pieces(first, 0);
#pragma unroll
      for (int part = 0; part < kValueParts; ++part) {
        const int index = part * kWave + lane;
        const int column = index / NVW;
        const int a = first - 63 + column;
        value_in[part] = (column < kBlockRows + kWave && a >= 1 && a <= view.len - 1)
            ? view.vbits[static_cast<int64_t>(a) * NVW + (index - column * NVW)] : 0u;
      }
    }
  };
  // What a chunk leaves in global memory (two row sums per row, its record) is held back
  // until the next chunk has started: nothing young is then in flight when a block waits for
  // its loads, which retire in order with every store and atomic issued before them.
  float pending_weight_sum = 0.0f, pending_numerator_sum = 0.0f;
  int pending_window = 0;
  uint32_t pending_kept = 0u;
  int pending_first = -1, pending_rows = 0;
  const auto flush_outputs = [&]() {
    if (pending_first < 0) return;
    // lanes 0..3 of every 16-lane group write the four rows of their group
    const int e = lane & 15;
    const int r = 4 * (lane >> 4) + e;
    if (e < 4 && r < pending_rows) {
      float4* row_stats = view.stats + (view.diag0 + 1 + pending_first + r);
      atomicAdd(&row_stats->y, pending_weight_sum);
      if (needs_utility) atomicAdd(&row_stats->z, pending_numerator_sum);
    }
    if (view.checkpoints != nullptr) {
      float* slot =
          view.checkpoints + static_cast<int64_t>(pending_first / kChunk) * view.record_floats;
      reinterpret_cast<uint16_t*>(slot + kWave)[lane] = static_cast<uint16_t>(pending_window);
      if constexpr (DROPOUT) {
        // the gradient pass reads the decisions back instead of hashing again
        reinterpret_cast<uint16_t*>(slot + kCheckpointFloats)[lane] =
            static_cast<uint16_t>(pending_kept);
      }
    }
    pending_first = -1;
  };
  issue_block_loads(0);
  for (int first = 0; first < view.steps; first += kBlockRows) {
    const int count = min(kBlockRows, view.steps - first);
    wave_lds_fence();
    if (lane < kBlockRows) {
      uint4* row_words = reinterpret_cast<uint4*>(rows + lane * kRowWords);
      row_words[0] = symbols_in;
      row_words[1] = make_uint4(__float_as_uint(fmaf(stat_in.x, kLog2e, stat_in.w)), 0u, 0u, 0u);
    }
    if (needs_utility) {
      store_pieces(0);
#pragma unroll
      for (int part = 0; part < kValueParts; ++part) {
        if (part * kWave + lane < (kBlockRows + kWave) * NVW) {
          value_columns[part * kWave + lane] = value_in[part];
        }
      }
#pragma unroll
      for (int group = kGradGroup; group < kGradParts; group += kGradGroup) {
        if (group * kWave >= pieces) break;  // wave-uniform
        load_pieces(first, group);
        __builtin_amdgcn_sched_barrier(0);
        store_pieces(group);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (first + kBlockRows < view.steps) issue_block_loads(first + kBlockRows);
    __builtin_amdgcn_sched_barrier(0);
    for (int local = 0; local < count; local += kChunk) {
      const int rows_here = min(kChunk, count - local);
      const int chunk_first = first + local;
      if (view.checkpoints != nullptr) {
        float* slot =
            view.checkpoints + static_cast<int64_t>(chunk_first / kChunk) * view.record_floats;
        slot[lane] = band.evidence;
      }
      flush_outputs();  // of the chunk before
      const int window_before = band.window - kCountBias;
      float peak_overflow = 0.0f;
      wave_lds_fence();
      if (needs_utility) {
        // (the widest tile in two batches: its registers decide a fourth wave per SIMD)
        utility_tiles_staged<NVW, DVP, false, (DVP > 32 ? 3 : 5)>(grads + local * grad_lds_pitch, grad_lds_pitch,
                                              P.grad_pitch / 32, value_columns + local * NVW,
                                              sign_table, utilities, kUtilityPitch, discard, lane);
        wave_lds_fence();
      }
      uint32_t kept_bits = 0u;  // bit r: this lane's pair of row r is kept
      v4f first_weight_sums;    // of rows 0 .. 7
      // compiled twice: once every lane is past its window fill no masking is needed
      auto run_chunk = [&](auto steady_tag, auto quiet_tag) {
        constexpr bool STEADY = decltype(steady_tag)::value;
        // QUIET (steady chunks only): no window of the chunk can get small enough for its
        // overflow term to reach `tail_threshold`, so the terms are left out (they could not
        // move a float32 result) and the window counts are only kept up to date: the
        // entering and the leaving mismatches are summed and applied after the chunk.
        constexpr bool QUIET = decltype(quiet_tag)::value;
        uint32_t entering = 0u, leaving = 0u;
        // quiet chunks carry 1 + S: one fused multiply-add per row, and the root below
        // needs no addition (the weight only sees S through sqrt(1 + S) anyway)
        float one_plus_evidence = 1.0f + band.evidence;
        const uint32_t* row = rows + local * kRowWords;
        if constexpr (QUIET) {
          // Quiet chunks, the common case, take their rows four at a time through each stage
          // (slides and gates, evidence and weights, hash rounds, stores): every stage then
          // offers the scheduler four independent dependency chains instead of one.
          constexpr int kGroup = 4;
          uint4 ahead_symbols[kGroup];
          float ahead_shift[kGroup], ahead_utility[kGroup];
          const auto fetch_group = [&](int g) {
#pragma unroll
            for (int j = 0; j < kGroup; ++j) {
              ahead_symbols[j] = *reinterpret_cast<const uint4*>(row + (g + j) * kRowWords);
              ahead_shift[j] = __uint_as_float(row[(g + j) * kRowWords + 4]);
              ahead_utility[j] = utilities[(g + j) * kUtilityPitch + lane];
            }
          };
          fetch_group(0);
#pragma unroll
          for (int g = 0; g < kChunk; g += kGroup) {
            float gates[kGroup], shifts[kGroup], group_utilities[kGroup];
            uint32_t hashes[kGroup];
#pragma unroll
            for (int j = 0; j < kGroup; ++j) {
              const uint4 words = ahead_symbols[j];
              shifts[j] = ahead_shift[j];
              group_utilities[j] = ahead_utility[j];
              band.key_word = dpp_wave_shr1(words.z, band.key_word);
              band.old_key_word = dpp_wave_shr1(words.w, band.old_key_word);
              const uint32_t differing = words.x ^ band.key_word;
              gates[j] = decay_of_biased_count(biased_popc(differing), P.gate_log2);
              entering = popc_plus(differing, entering);
              leaving = popc_plus(words.y ^ band.old_key_word, leaving);
              if constexpr (DROPOUT) {
                route_hash = dpp_wave_shr1(route_hash_of(chunk_first + g + j + 1), route_hash);
                hashes[j] = route_hash;
              }
            }
            if (g + kGroup < kChunk) fetch_group(g + kGroup);
            __builtin_amdgcn_sched_barrier(0);
            float group_weights[kGroup];
#pragma unroll
            for (int j = 0; j < kGroup; ++j) {
              one_plus_evidence = fmaf(gates[j], one_plus_evidence, 1.0f);
              group_weights[j] =
                  fast_exp2(fmaf(fast_sqrt(one_plus_evidence), logit_gain, -shifts[j]));
            }
            bool kept[kGroup];
            if constexpr (DROPOUT) {
              __builtin_amdgcn_sched_barrier(0);
              uint32_t states[kGroup];
#pragma unroll
              for (int j = 0; j < kGroup; ++j) {
                const int t = view.diag0 + 1 + chunk_first + g + j;
                states[j] = hashes[j] ^ fold16(static_cast<uint32_t>(t) ^ 0xb5297a4du);
              }
              const uint32_t round_keys[4] = {key.head_key, key.batch_key, key.seed_low_key,
                                              key.seed_high_key};
#pragma unroll
              for (int round = 0; round < 4; ++round) {
#pragma unroll
                for (int j = 0; j < kGroup; ++j) states[j] = open_round(states[j]) ^ round_keys[round];
              }
#pragma unroll
              for (int j = 0; j < kGroup; ++j) kept[j] = fold16(open_round(states[j])) >= key.keep_from;
              __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < kGroup; ++j) {
              float dropped_utility = group_weights[j] * group_utilities[j];
              if constexpr (DROPOUT) {
                dropped_utility = kept[j] ? dropped_utility : 0.0f;
                kept_bits = doubled_plus_flag(kept_bits, kept[j]);
              }
              weights[((g + j) & (kWeightRows - 1)) * kWeightPitch + lane] = group_weights[j];
              utilities[(g + j) * kUtilityPitch + lane] = dropped_utility;
            }
            if (g + kGroup == kWeightRows) {
              wave_lds_fence();
              first_weight_sums = tile_row_sums<kWeightRows>(weights, kWeightPitch, lane);
              wave_lds_fence();
            }
          }
          band.window += static_cast<int>(entering - leaving);
          band.evidence = one_plus_evidence - 1.0f;  // exact: 1 <= 1 + S
          if constexpr (DROPOUT) kept_bits = __builtin_bitreverse32(kept_bits) >> 16;  // bit r: row r
          return;
        }
        uint4 next_symbols = *reinterpret_cast<const uint4*>(row);
        float next_shift = __uint_as_float(row[4]);
        float next_utility = utilities[lane];
#pragma unroll
        for (int r = 0; r < kChunk; ++r) {
          const RowSymbols symbols{next_symbols.x, next_symbols.y, next_symbols.z, next_symbols.w};
          const float shift = next_shift;
          const float utility = next_utility;
          if (r + 1 < kChunk) {  // the next row's words are on their way while this one runs
            next_symbols = *reinterpret_cast<const uint4*>(row + (r + 1) * kRowWords);
            next_shift = __uint_as_float(row[(r + 1) * kRowWords + 4]);
            next_utility = utilities[(r + 1) * kUtilityPitch + lane];
          }
          const int i = min(chunk_first + r, last_step);
          const int t = view.diag0 + 1 + i;
          StepOut s;
          if constexpr (QUIET) {
            band.key_word = dpp_wave_shr1(symbols.key, band.key_word);
            band.old_key_word = dpp_wave_shr1(symbols.old_key, band.old_key_word);
            const uint32_t differing = symbols.query ^ band.key_word;
            const float gate = decay_of_biased_count(biased_popc(differing), P.gate_log2);
            one_plus_evidence = fmaf(gate, one_plus_evidence, 1.0f);
            entering = popc_plus(differing, entering);
            leaving = popc_plus(symbols.old_query ^ band.old_key_word, leaving);
            s.active = true;
          } else {
            s = forward_step<NVW, STEADY, false, true>(band, symbols, i, lane, W, P.gate_log2);
            peak_overflow = fmaxf(peak_overflow, s.overflow);
          }
          // (outside quiet chunks the root is formed exactly as the gradient pass forms it:
          // with long matches the logits are large, and a last-bit difference between the
          // two passes' roots would show in the normalisation)
          float root;
          if constexpr (QUIET) {
            root = fast_sqrt(one_plus_evidence);
          } else {
            const float one_plus = 1.0f + s.evidence;
            root = one_plus * fast_rsq(one_plus);
          }
          const bool live = STEADY || (s.active && r < rows_here);
          const float weight = live ? fast_exp2(fmaf(root, logit_gain, -shift)) : 0.0f;
          // (the factor 1 / (1 - p) of the kept pairs is applied to the row sums)
          float dropped_utility = weight * utility;
          if constexpr (DROPOUT) {
            route_hash = dpp_wave_shr1(route_hash_of(i + 1), route_hash);
            set_row(key, t);
            const bool kept = dropout_keeps(key, route_hash);
            dropped_utility = kept ? dropped_utility : 0.0f;
            kept_bits = doubled_plus_flag(kept_bits, kept);  // rows end up in reverse order
          }
          weights[(r & (kWeightRows - 1)) * kWeightPitch + lane] = weight;
          utilities[r * kUtilityPitch + lane] = dropped_utility;
          if (r + 1 == kWeightRows) {
            wave_lds_fence();
            first_weight_sums = tile_row_sums<kWeightRows>(weights, kWeightPitch, lane);
            wave_lds_fence();
          }
        }
        if constexpr (QUIET) {
          band.window += static_cast<int>(entering - leaving);
          band.evidence = one_plus_evidence - 1.0f;  // exact: 1 <= 1 + S
        }
        if constexpr (DROPOUT) kept_bits = __builtin_bitreverse32(kept_bits) >> 16;  // bit r: row r
      };
      if (chunk_first >= W + kWave && rows_here == kChunk) {
        // a window loses at most D mismatches per row
        const bool quiet = __ballot(window_before < quiet_window) == 0ull;
        if (quiet) {
          run_chunk(std::true_type{}, std::true_type{});
        } else {
          run_chunk(std::true_type{}, std::false_type{});
        }
      } else {
        run_chunk(std::false_type{}, std::false_type{});
      }
      wave_lds_fence();
      {
        // the second half of the weight tile repeats as rows 8 .. 15 of the product, which is
        // where the lanes of groups 2 and 3 expect the sums of the chunk's rows 8 .. 15
        const v4f second_weight_sums = tile_row_sums<kWeightRows>(weights, kWeightPitch, lane);
        const v4f weight_sums = lane < 32 ? first_weight_sums : second_weight_sums;
        const v4f numerator_sums = tile_row_sums<kChunk>(utilities, kUtilityPitch, lane);
        const int e = lane & 15;
        pending_weight_sum = e == 0 ? weight_sums[0] : e == 1 ? weight_sums[1]
                           : e == 2 ? weight_sums[2] : weight_sums[3];
        pending_numerator_sum = e == 0 ? numerator_sums[0] : e == 1 ? numerator_sums[1]
                              : e == 2 ? numerator_sums[2] : numerator_sums[3];
        if constexpr (DROPOUT) pending_numerator_sum *= P.inverse_keep;
      }
      // bit 15 of the window word tells the gradient pass that some overflow term
      // of the chunk is large enough to matter
      const bool noisy = __ballot(peak_overflow >= P.tail_threshold) != 0ull;
      // The gradient pass carries its gate adjoints in two bfloat16 terms unless matches get
      // long: their adjoints are much larger than the gradient sums they cancel in.  Evidence
      // of kLongMatchEvidence at a chunk's end takes an exact match of at least that many rows
      // (random symbols of eight bits never reach it).  Header word 4; every writer writes 1.
      const bool long_match = __ballot(band.evidence >= kLongMatchEvidence) != 0ull;
      if ((noisy || long_match) && lane == 0) P.work_counter[3] = 1;
      pending_window = min(window_before, kRecordWindowMax) | (noisy ? 0x8000 : 0);
      pending_kept = kept_bits;
      pending_first = chunk_first;
      pending_rows = rows_here;
    }
  }
  flush_outputs();
}

// Gradient pass.  Persistent blocks pull bands from a work counter.  A band is
// processed from its last row upwards because the gate adjoint
//   h(n) = b(n) (S(n) + overflow(n)) - sum_{m=n..n+W} b(m) overflow(m),
//   b(n) = A(n) + gate(n+1) b(n+1)
// needs the adjoints of later rows, while S needs earlier rows.  S is
// therefore rebuilt from checkpoints: one cheap forward sweep per band stores
// (S, window) once per LDS-staged segment, one per segment stores them every kChunk
// rows in LDS, and each chunk is then replayed forward into registers and
// walked backwards.  The windowed sum of b*overflow lives in a ring of W+1
// rows in global memory that is touched only while some overflow term of the
// wave is above `tail_threshold` (long near-exact matches).
//
// Each chunk leaves its route weights d*p and gate adjoints h in LDS as
// [row][lane] tiles (with zero margins), from which the three contractions
//   dV[a, :]   += sum_t  d p(t, a) go[t, :]
//   dK[a-1, :] += c sum_t h(t, a) z(q[t, :])
//   dQ[t, :]   += c sum_a h(t, a) z(k[a-1, :]),   c = mismatch_scale / (2 D)
// are formed on the matrix cores (v_mfma_f32_16x16x32_bf16, split operands).  In the chunk's own
// (row r, window column c) coordinates the pair (r, lane l) sits at
// c = 64 - l + r, i.e. the tile read with a skew is an ordinary matrix.  The
// window spans 80 columns = 5 MFMA tiles; a chunk completes exactly the last
// tile (the 16 highest columns), which is flushed with global atomics, and the
// other four shift up by one tile for the next chunk, so column sums live in
// accumulator registers for their whole life.
// The tile is stored by window column: pair (r, lane l) at [r][c], c = 64 - l + r, so row r
// holds its 64 pairs in columns r + 1 .. r + 64 and zeros elsewhere.  Pitch 84: with
// 4 * pitch = 16 (mod 64) the reads of the column sums (lane (li, lg) reads rows
// 4 lg .. 4 lg + 3 of column li) touch 64 different LDS banks, and the row sums read four
// neighbouring columns of row li as one aligned 16-byte word, rows 20 (mod 64) banks apart.
constexpr int kTilePitch = 84;
constexpr int kCheckpointChunksMax = 4;  // chunks per staged segment at most
constexpr int kWindowTiles = 5;  // 80 window columns

// -1.0f where symbol bit `bit` of `word` is set, +1.0f where it is clear: the negated
// symbol, two instructions; callers fold the sign into their output scale.  Columns
// beyond the symbol width produce values nobody stores.
__device__ __forceinline__ float negated_symbol(uint32_t word, int bit) {
  return sign_from_bit31(word << (31 - bit));
}

// register budget of the gradient kernel: waves per SIMD it is compiled for.  Its time falls
// almost in proportion to the waves that share a SIMD; one value tile and one symbol tile
// fit three (168 registers) without a spill.
// The form that walks pieces of bands (PIECES of vjp_gradients_kernel) decides per chunk
// whether the accumulators move; the copies that takes do not fit the two tightest budgets,
// which give up a wave per SIMD rather than spill (that form runs only when there are too
// few bands to fill the SIMDs anyway).
constexpr int gradient_waves(int value_tiles, int symbol_tiles, bool pieces = false) {
  if (value_tiles == 1 && symbol_tiles == 1) return pieces ? 2 : 3;
  if (value_tiles == 4 && symbol_tiles == 2) return 1;   // 120 accumulator registers alone
  if (value_tiles == 4 && pieces) return 1;
  return 2;
}

// rows staged in LDS per segment of the gradient kernel (a multiple of kChunk): with 32 a
// single-wave block of the narrowest tile needs 11.4 KB, which leaves room for three per SIMD
constexpr int gradient_segment(int /*dvp*/) { return 32; }

// Waves per block of the gradient kernel.  The waves of a block own neighbouring bands of
// one (sequence, head) and walk them in step: at the same band-local step every band
// completes the same 16 columns, so the column sums of all bands are added in LDS and leave
// in one set of global atomics; the rows of a band are the rows its neighbour (64 diagonals
// further) handles four chunks later, so row sums travel from band to band through a short
// LDS queue and only the last band adds them to memory.  Global float atomics are bounded
// by the number of 64-byte row segments they touch (about 21 G segments per second on the
// whole chip, whatever the number of lanes), which made them the limit of the wide tiles.
constexpr int kQueueSlots = 4;  // a row tile is read four chunks after it was written: the
                                // reader takes it before the barrier, the writer refills the
                                // slot behind the barrier

// LDS bytes of a block of the gradient kernel up to which four blocks share a compute unit;
// the queues of row tiles are kept where the block stays within them
constexpr size_t kGradientBlockLdsBudget = 40 * 1024;

// floats of the shared LDS area of a block before the exchange tiles: window columns and,
// with several waves, the work index
constexpr int gradient_shared_fixed_floats(int segment, int value_words_per_column, int waves) {
  return (segment + kWave) * (2 + value_words_per_column) + (waves > 1 ? 64 : 0);
}

// floats of a 16 x 16 accumulator tile on its way through LDS (lane (li, lg) owns rows
// 4 lg .. 4 lg + 3 of column li): all 64 lanes, or the 32 lanes of columns 0 .. 7 when no
// tile has more than 8 live columns
constexpr int exchange_tile_floats(bool narrow) { return narrow ? 2 * kWave : 4 * kWave; }

// bfloat16 elements of padding per staged grad_output row (none at the narrowest width,
// where the block's LDS decides how many blocks a compute unit holds)
constexpr int gradient_row_padding(int dvp) { return dvp > 8 ? 8 : 0; }

constexpr int kRestPitch = 84;  // 16-bit elements per row of the third-term plane

// LDS floats a wave of the gradient kernel owns: tile, row words, query words, sink, sign
// table, third-term plane and the staged grad_output rows (bfloat16 terms, `grad_pitch`
// elements per row plus padding), in whole 16-byte units
constexpr size_t gradient_wave_floats(int dvp, int grad_pitch) {
  const size_t segment = gradient_segment(dvp);
  const size_t fixed = kChunk * kTilePitch + segment * kRowWords + segment + kWave +
                       kSignTableWords + kChunk * kRestPitch / 2;
  return (fixed + (segment * (grad_pitch + gradient_row_padding(dvp)) + 1) / 2 + 3) / 4 * 4;
}

// One step of the reverse recurrence b = adjoint + gate * b_below with the carry held as
// two floats: returns the float32 sum and updates `rest`, what the additions so far have
// lost.  The lost part of this step's addition is taken by the three-operation form that
// is exact when the carried product is the larger operand: that is the case that matters
// (a long sum next to one more term), and in the other case what it leaves out is of the
// size of one ordinary rounding.  The product's own rounding is left alone: along an exact
// match the gate is 1, elsewhere the gates shrink old errors geometrically.
__device__ __forceinline__ float carry_step(float gate, float below, float adjoint, float& rest) {
  const float product = __fmul_rn(gate, below);  // (not contracted with the addition below)
  const float sum = __fadd_rn(product, adjoint);
  const float sum_rest = __fsub_rn(adjoint, __fsub_rn(sum, product));
  rest = fmaf(gate, rest, sum_rest);
  return sum;
}

// TERMS: bfloat16 terms that carry a gate adjoint into the symbol contractions.  Two terms
// hold it to 2^-18 of its size, which is enough where the terms of a gradient sum are of the
// size of the sum.  Long matches make them much larger than the sum (a row's adjoints
// cancel), so a launch in which the row-statistics pass has met a long match (evidence of
// kLongMatchEvidence at the end of a chunk, or an overflow term that matters: header word 4)
// runs the three-term form, 2^-21 by truncation; both forms are launched and the one that
// does not apply returns at once.
// PIECES: bands are cut into pieces (see the work items below); compiled apart, because the
// few extra live values cost the narrowest tile its third wave per SIMD.
template <int NVW, int DVP, int DT, bool VARLEN, bool DROPOUT, int NW, int TERMS, bool PIECES>
__global__ __launch_bounds__(kWave * NW)
__attribute__((amdgpu_waves_per_eu(gradient_waves((DVP + 15) / 16, DT, PIECES))))
void vjp_gradients_kernel(VjpParams P) {
  static_assert(NW == 1 || NW == 2, "blocks of one or two waves");
  static_assert(TERMS == 2 || TERMS == 3, "two or three terms per gate adjoint");
  static_assert(!PIECES || NW == 1, "pieces of bands are walked by single-wave blocks");
  if ((P.header[4] != 0) != (TERMS == 3)) return;
  constexpr int VT = (DVP + 15) / 16;   // value-dimension MFMA tiles
  constexpr bool kFetchAhead = true;  // row words and operands are fetched ahead of their use
  constexpr int SEG = gradient_segment(DVP);  // rows staged in LDS at a time
  constexpr int SEG_CHUNKS = SEG / kChunk;
  extern __shared__ float lds_all[];
  // LDS: first what the waves of a block share, then one region per wave.  Shared are the
  // window columns of a segment (every band of the block meets the same columns at the same
  // band-local step; each wave stores them, with the same values), the work index, the
  // column tiles on their way to wave 0 and the queues of row tiles.
  const int wave = NW > 1 ? __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6) : 0;
  const bool row_queue_on = NW > 1 && P.row_queue != 0;
  constexpr int kSharedFixed = gradient_shared_fixed_floats(SEG, NVW, NW);
  uint32_t* key_window = reinterpret_cast<uint32_t*>(lds_all);  // [SEG + 64] key words of the columns
  uint32_t* old_key_window = key_window + SEG + kWave;       // [SEG + 64] key words of the columns
                                                             // W + 1 to the left
  uint32_t* value_window = old_key_window + SEG + kWave;     // [SEG + 64][NVW] value sign words
  int* shared_unit = reinterpret_cast<int*>(value_window + (SEG + kWave) * NVW);  // [2] (+ padding)
  float* lds = lds_all + kSharedFixed + wave * P.wave_lds_floats;  // this wave's own region
  float* column_exchange = lds_all + kSharedFixed + NW * P.wave_lds_floats;
                                                    // [NW - 1][VT + DT][exchange_tile_floats]
  float* row_queue = column_exchange + (NW - 1) * (VT + DT) * P.exchange_tile_floats;
                                                    // [NW - 1][kQueueSlots][DT][exchange_tile_floats]
  float* tile = lds;                                         // [kChunk][kTilePitch]
  uint32_t* tile_bits = reinterpret_cast<uint32_t*>(tile);   // the same tile as split operands
  uint32_t* rows = reinterpret_cast<uint32_t*>(tile + kChunk * kTilePitch);  // [SEG][kRowWords]
  uint32_t* query_rows = rows + SEG * kRowWords;             // [SEG] query words of the rows
  float* discard = reinterpret_cast<float*>(query_rows + SEG); // [64] sink of the utility tile
  uint32_t* sign_table = reinterpret_cast<uint32_t*>(discard + kWave);  // [kSignTableWords]
  // third bfloat16 term of the gate adjoints, [kChunk][kRestPitch], same geometry as `tile`
  uint16_t* rest_plane = reinterpret_cast<uint16_t*>(sign_table + kSignTableWords);
  // [SEG][GP] bfloat16 terms of the grad_output rows (GP elements per row: the terms in
  // whole 32-element blocks, plus 16 bytes against bank conflicts where LDS allows)
  uint16_t* grad_rows_lds = rest_plane + kChunk * kRestPitch;
  const int GP = P.grad_pitch + gradient_row_padding(DVP);
  const int grad_chunks = P.grad_pitch / 8;   // 16-byte pieces per row
  constexpr int kGradChunksMax = grad_term_pitch(kMaxGradTerms, DVP) / 8;

  // The kernel has no registers for the many addresses and offsets that derive from the
  // lane number alone (the compiler hoists them out of all loops: fifty registers of the
  // narrowest tile, spills in the wide ones): the lane number is made opaque once per
  // chunk, so that they are recomputed where they are used.  That costs the narrowest tile
  // 3 % more instructions and gives it its third wave per SIMD.
  constexpr bool kRecomputeLaneValues = true;
  // completed tiles wait in registers for the next chunk's replay to cover their atomics
  constexpr bool kFlushAtOnce = false;
  const int lane_id = threadIdx.x & (kWave - 1);
  int lane = lane_id;
  int li = lane & 15;   // MFMA row (A) / column (B, C) index
  int lg = lane >> 4;   // MFMA k index (A, B) / row group (C)
  const int W = P.L.W;
  const int D = P.L.D;
  const int Dv = P.L.Dv;
  const bool want_q = (P.gradient_mask & ROSA_GRAD_QUERY) != 0;
  const bool want_k = (P.gradient_mask & ROSA_GRAD_KEY) != 0;
  const bool want_v = (P.gradient_mask & ROSA_GRAD_VALUE) != 0;
  const bool want_qk = want_q || want_k;
  const float adjoint_gain = 0.5f * kSqrtScale * P.scale;  // scale * U'(S) * sqrt(1 + S)
  const float logit_gain = in_vector_register(P.logit_gain);
  const float inverse_keep = in_vector_register(P.inverse_keep);
  // the contractions run on negated symbols
  // dQ and dK are linear in the route adjoints, so the constant factor of every adjoint
  // (adjoint_gain) is applied here, once per flushed element, instead of once per pair
  const float symbol_scale = -0.5f * P.mismatch_scale / static_cast<float>(D) * adjoint_gain;
  float* ring = P.block_scratch +
      (static_cast<int64_t>(blockIdx.x) * NW + wave) * P.block_scratch_floats;
  // without chunk records: (S, window) before every chunk of the current segment, then
  // before every segment of the band
  // (three-term form) what the float32 ring terms do not hold of (b + rest) * overflow, as
  // bfloat16: the second float of the windowed sum
  [[maybe_unused]] uint16_t* ring_low =
      reinterpret_cast<uint16_t*>(ring + static_cast<int64_t>(P.ring_rows) * kWave);
  float* ck_evidence = ring + static_cast<int64_t>(P.ring_rows) * (kWave + kWave / 2);  // [SEG_CHUNKS][64]
  int* ck_window = reinterpret_cast<int*>(ck_evidence + SEG_CHUNKS * kWave);
  // without records, two levels of (S, window) checkpoints: before every group of
  // `segment_group` segments of the band (one forward sweep over the band), and before every
  // segment of the group the reverse walk is in (one more sweep over that group)
  float* group_ck = ck_evidence + 2 * kCheckpointChunksMax * kWave;  // [group][(S, window)][64]
  const int G = P.segment_group;

  // zero the tile once: its margins are never written again
  for (int index = lane; index < kChunk * kTilePitch; index += kWave) tile[index] = 0.0f;
  for (int index = lane; index < kChunk * kRestPitch; index += kWave) rest_plane[index] = 0;
  fill_sign_table(sign_table, lane);
  wave_lds_fence();

  int pulls = 0;
  for (;;) {
    int unit_index = 0;
    if constexpr (NW == 1) {
      if (lane == 0) unit_index = atomicAdd(P.work_counter, 1);
    } else {
      // one pull per block; the two slots alternate, so that a wave that is still reading
      // the previous index is not overtaken by the next pull
      if (threadIdx.x == 0) shared_unit[pulls & 1] = atomicAdd(P.work_counter, 1);
      block_barrier();
      unit_index = shared_unit[pulls & 1];
      ++pulls;
    }
    unit_index = __builtin_amdgcn_readfirstlane(unit_index);
    if (unit_index >= P.total_units) break;
    // The unit names the first band of the block's group of NW neighbouring bands (the
    // longest of them); wave w takes band w of the group.  Everything that decides how often
    // the block meets at a barrier derives from the first band, which all waves know.
    // With long bands and few of them a band is cut into pieces of `piece_rows` rows that
    // different waves take (work item = band * max_pieces + piece): the kernel would otherwise
    // last as long as its longest band.  The gate adjoints have a finite horizon (a row's
    // adjoint depends on the route adjoints of the W - 1 rows below it only), so a piece
    // starts its reverse walk that many rows below its last row, with an empty carry and an
    // empty window sum, and takes only the recurrences from those rows; its forward state
    // comes from the chunk records (or the forward sweeps) like that of a whole band.
    const int piece = PIECES ? unit_index % P.max_pieces : 0;
    const Unit lead = decode_unit<VARLEN>(P.L, PIECES ? unit_index / P.max_pieces : unit_index);
    if (!lead.valid) continue;
    if (NW > 1 && lead.block % NW != 0) continue;
    const int band_rows = lead.len - 1 - lead.block * kWave;
    if (band_rows <= 0) continue;
    Unit u = lead;
    u.block += wave;
    BandView view;
    int hv;
    const bool have_band = make_view<NVW, VARLEN>(P, u, view, hv);
    // rows [row_begin, row_end) are this work item's; the walk starts at row my_steps - 1
    int row_begin = 0, row_end = have_band ? view.steps : 0;
    int my_steps = row_end;  // a wave without a band only keeps step
    if constexpr (PIECES) {
      row_begin = piece * P.piece_rows;
      if (row_begin >= view.steps) continue;
      row_end = min(view.steps, row_begin + P.piece_rows);
      const int halo = (P.gradient_mask & (ROSA_GRAD_QUERY | ROSA_GRAD_KEY)) != 0
          ? (P.L.W - 1 + kChunk - 1) / kChunk * kChunk : 0;
      my_steps = min(view.steps, row_end + halo);
    }
    const int lead_steps = PIECES ? my_steps : band_rows;
    DropoutKey key;
    if constexpr (DROPOUT) {
      key = make_dropout_key(static_cast<uint64_t>(*P.dropout_seed), u.head, u.seq, P.dropout_p);
    }

    // column accumulators of the 80-column window, one MFMA tile per 16 columns
    v4f value_acc[kWindowTiles][VT];
    v4f key_acc[kWindowTiles][DT];
#pragma unroll
    for (int m = 0; m < kWindowTiles; ++m) {
#pragma unroll
      for (int n = 0; n < VT; ++n) value_acc[m][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int n = 0; n < DT; ++n) key_acc[m][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }

    const int lead_segments = (lead_steps + SEG - 1) / SEG;
    const int segments = (my_steps + SEG - 1) / SEG;
    Band<NVW> band;
    // Without stored checkpoints, a band-level forward sweep leaves (S, window) before the
    // first row of every segment and a segment-level one before every chunk.
    const bool stored = have_band && view.checkpoints != nullptr;
    const int groups = (segments + G - 1) / G;
    float* seg_ck = group_ck + static_cast<int64_t>(2 * groups) * kWave;  // [segment of the group]
    // sweep over segments [from, to) starting from `band`, leaving the state before each of
    // them where `keep` says; the state after the last one is not needed
    const auto sweep_segments = [&](int from, int to, auto keep) {
      load_sliding<NVW>(band, view, from * SEG, lane, W);
      for (int segment = from; segment < to; ++segment) {
        keep(segment);
        if (segment + 1 == to) break;
        const int first = segment * SEG;
        wave_lds_fence();
        stage_rows<NVW, kRowSymbols>(view, first, SEG, lane, rows, W);
        wave_lds_fence();
        sweep_rows<NVW>(band, rows, first, SEG, lane, W, P.gate_log2);
      }
    };
    if (have_band && !stored && segments > 1) {
      band.evidence = 0.0f;
      band.window = 0;
      // (the sweep ends with the last group's first segment: nothing later is kept)
      sweep_segments(0, (groups - 1) * G + 1, [&](int segment) {
        if (segment % G == 0) {
          group_ck[(2 * (segment / G)) * kWave + lane] = band.evidence;
          group_ck[(2 * (segment / G) + 1) * kWave + lane] = __int_as_float(band.window);
        }
      });
    }

    // reverse state carried across chunks and segments
    float adjoint_carry = 0.0f;   // b of the row below on this diagonal
    // what the float32 additions of the carry have lost so far (three-term form only): along
    // an exact match the gates are 1 and b is a running sum of hundreds of route adjoints of
    // both signs, whose rounding would otherwise cost periodic inputs their margin
    [[maybe_unused]] float carry_rest = 0.0f;
    float gate_below = 0.0f;      // gate of the row below
    float ring_sum = 0.0f;        // sum of b * overflow over the next W + 1 rows
    // what ring_sum has lost and the sum of the terms' low parts (three-term form): h is the
    // difference of b (S + o) and this sum, both hundreds of adjoints large along an exact
    // match longer than the window, so both are carried as two floats
    [[maybe_unused]] float ring_sum_low = 0.0f;
    int ring_live = 0;            // rows for which the ring still holds non-zero terms
    int ring_fresh = 0;           // ring reads that must be treated as zero
    const int last_step = my_steps - 1;
    // The global atomics of a chunk are issued one chunk later, right before the next
    // chunk's replay, so that their latency is covered by arithmetic instead of being
    // waited for at the next chunk's first register reuse.
    v4f done_value[VT];
    v4f done_key[DT];
    v4f done_query[DT];
    int done_first = -1;  // first step of the chunk whose results are pending (-1: none)
    int done_rows = 0;
    // which of the pending results this wave adds to memory itself (in a block of two waves
    // the value column sums leave through wave 0, the key column sums through wave 1, and
    // row sums through the last band that holds the rows)
    bool done_flush_value = true;
    bool done_flush_key = true;
    bool done_flush_rows = true;
    [[maybe_unused]] bool done_has_rows = true;  // false for the column tiles a piece flushes when it ends
    // step 0 of the band: row diag0 + 1 (query gradients), column 1 (value gradients, key
    // position 0)
    const uint32_t symbol_stride = P.symbols_by_head ? D : static_cast<uint32_t>(P.L.H) * D;
    const uint32_t value_stride =
        P.values_by_head ? P.value_stride : static_cast<uint32_t>(P.L.Hv) * P.value_stride;
    float* band_query_base = P.symbols_by_head
        ? P.grad_query + (u.word_base + view.diag0) * D
        : P.grad_query + ((static_cast<int64_t>(u.start) + view.diag0 + 1) * P.L.H + u.head) * D;
    float* band_key_base = P.symbols_by_head
        ? P.grad_key + u.word_base * D
        : P.grad_key + (static_cast<int64_t>(u.start) * P.L.H + u.head) * D;
    // (sequence, value head, position 0) in a head-major tensor over the value heads
    const int64_t value_run = VARLEN ? static_cast<int64_t>(hv) * P.L.N + u.start
                                     : (static_cast<int64_t>(u.seq) * P.L.Hv + hv) * P.L.T;
    float* band_value_base = P.values_by_head
        ? P.grad_value + value_run * P.value_stride
        : P.grad_value +
              ((static_cast<int64_t>(u.start) + 1) * P.L.Hv + hv) * P.value_stride + P.value_offset;
    // One completed 16 x 16 tile: lane (li, lg) holds rows 4 lg .. 4 lg + 3 of column li.
    // With at most 8 live columns the upper half of every 16 lanes takes the odd rows from the
    // lower half, so that two instructions carry what would otherwise take four and each of
    // them covers pairs of neighbouring rows (one 64-byte segment in a head-major accumulator).
    // `base` (element (row 0, column 0) of the tile) and `row_stride` are wave-uniform, so
    // the address of a lane is a scalar pointer plus a 32-bit lane offset; FULL tiles (every
    // row exists) need no row test.
    auto add_tile = [&](auto full_tag, float* base, uint32_t row_stride, int columns, v4f values,
                        float scale, int rows_left) {
      constexpr bool FULL = decltype(full_tag)::value;
      // rows_left: valid rows counted from row 4 lg
      if (columns <= 8) {
        const int half = li >> 3;
        const float first = dpp_row_shr8(values[0], values[1]);   // rows 4 lg, 4 lg + 1
        const float second = dpp_row_shr8(values[2], values[3]);  // rows 4 lg + 2, 4 lg + 3
        if ((li & 7) < columns) {
          const uint32_t offset = static_cast<uint32_t>(4 * lg + half) * row_stride + (li & 7);
          if (FULL || half < rows_left) atomicAdd(base + offset, scale * first);
          if (FULL || 2 + half < rows_left) {
            atomicAdd(base + 2 * row_stride + offset, scale * second);
          }
        }
      } else if (li < columns) {
        const uint32_t offset = static_cast<uint32_t>(4 * lg) * row_stride + li;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (FULL || e < rows_left) atomicAdd(base + e * row_stride + offset, scale * values[e]);
        }
      }
    };
    auto issue_pending = [&]() {
      if (done_first < 0) return;
      // wave-uniform element (row 0, column 0) of the three tiles: the band's bases moved
      // by the chunk's first step
      const uint64_t symbol_step =
          static_cast<uint64_t>(static_cast<uint32_t>(done_first)) * symbol_stride;
      float* query_base = band_query_base + symbol_step;
      float* key_base = band_key_base + symbol_step;
      float* value_base =
          band_value_base + static_cast<uint64_t>(static_cast<uint32_t>(done_first)) * value_stride;
      const auto add_all = [&](auto full_tag, int rows_left, int columns_left) {
        if (want_q && (!PIECES || done_has_rows) && (NW == 1 || done_flush_rows)) {
#pragma unroll
          for (int n = 0; n < DT; ++n) {
            add_tile(full_tag, query_base + 16 * n, symbol_stride, D - 16 * n, done_query[n],
                     symbol_scale, rows_left);
          }
        }
        if (want_v && (NW == 1 || done_flush_value)) {
#pragma unroll
          for (int n = 0; n < VT; ++n) {
            add_tile(full_tag, value_base + 16 * n, value_stride, Dv - 16 * n, done_value[n], 1.0f,
                     columns_left);
          }
        }
        if (want_k && (NW == 1 || done_flush_key)) {
#pragma unroll
          for (int n = 0; n < DT; ++n) {
            add_tile(full_tag, key_base + 16 * n, symbol_stride, D - 16 * n, done_key[n],
                     symbol_scale, columns_left);
          }
        }
      };
      if (done_rows == kChunk) {  // then every row and column of the chunk exists
        add_all(std::true_type{}, kChunk, kChunk);
      } else {
        const int columns = min(kChunk, view.len - 1 - done_first);  // columns a <= len - 1
        add_all(std::false_type{}, done_rows - 4 * lg, columns - 4 * lg);
      }
      done_first = -1;
    };

    // Chunk records written by the row-statistics pass, (S, window) before the chunk and
    // with dropout its keep decisions: each is fetched one chunk ahead of its use.
    float record_evidence = 0.0f;
    int record_window = 0;
    uint32_t record_kept = 0u;
    const auto fetch_record = [&](int chunk_index) {
      const float* slot =
          view.checkpoints + static_cast<int64_t>(chunk_index) * view.record_floats;
      record_evidence = slot[lane];
      record_window = reinterpret_cast<const uint16_t*>(slot + kWave)[lane];
      if constexpr (DROPOUT) {
        record_kept = reinterpret_cast<const uint16_t*>(slot + kCheckpointFloats)[lane];
      }
    };
    if (stored) fetch_record((my_steps - 1) / kChunk);

    for (int segment = lead_segments - 1; segment >= (PIECES ? row_begin / SEG : 0); --segment) {
      const int seg_first = segment * SEG;
      const int seg_last = min(my_steps, seg_first + SEG);
      // chunks of the first band in this segment: the trip count of every wave
      const int chunks = (min(lead_steps, seg_first + SEG) - seg_first + kChunk - 1) / kChunk;
      const bool segment_active = NW == 1 || seg_first < my_steps;
      if (segment_active) {
      if (!stored) {
        if (segments > 1) {
          if (segment == segments - 1 || segment % G == G - 1) {
            // the walk enters a group: the state before each of its segments up to this one
            const int group = segment / G;
            band.evidence = group_ck[(2 * group) * kWave + lane];
            band.window = __float_as_int(group_ck[(2 * group + 1) * kWave + lane]);
            sweep_segments(group * G, segment + 1, [&](int inner) {
              seg_ck[(2 * (inner % G)) * kWave + lane] = band.evidence;
              seg_ck[(2 * (inner % G) + 1) * kWave + lane] = __int_as_float(band.window);
            });
          }
          band.evidence = seg_ck[(2 * (segment % G)) * kWave + lane];
          band.window = __float_as_int(seg_ck[(2 * (segment % G) + 1) * kWave + lane]);
        } else {
          band.evidence = 0.0f;
          band.window = 0;
        }
        load_sliding<NVW>(band, view, seg_first, lane, W);
        // taken in here: a load left pending on this rarely taken path would make later
        // writes of these registers wait for every memory operation in flight
        asm volatile("" : : "v"(band.key_word), "v"(band.old_key_word));
      }
      // one round trip brings in everything the segment needs
      wave_lds_fence();
      // (all but the tightest variant: packed, Dv = 64, one wave per block has no registers
      // for it and stages array by array, which took a quarter of the kernel at Dv = 64)
      constexpr bool kHeavy = VT > 2 && VARLEN && NW == 1;
      if constexpr (!kHeavy) {
        // Every global load of the segment is issued before the first of them is used, so
        // the segment costs one memory latency (two when the grad_output rows need the
        // registers of the other arrays), not one per staged array.
        const bool row_lane = lane < SEG;
        const int i = min(seg_first + lane, view.steps - 1);  // rows past the end repeat the last
        const int t = view.diag0 + 1 + i;
        uint4 symbols = make_uint4(0u, 0u, 0u, 0u);
        uint4 record = make_uint4(0u, 0u, 0u, 0u);
        if (row_lane) {
          symbols.x = view.q[t];
          symbols.y = (t - W - 1 >= 0) ? view.q[t - W - 1] : 0u;
          symbols.z = view.k[i];
          symbols.w = (i - W - 1 >= 0) ? view.k[i - W - 1] : 0u;
          record = reinterpret_cast<const uint4*>(view.stats)[t];  // finalised
        }
        constexpr int kKeyParts = (SEG + 2 * kWave - 1) / kWave;
        uint32_t key_in[kKeyParts], old_key_in[kKeyParts];
#pragma unroll
        for (int part = 0; part < kKeyParts; ++part) {
          const int a = seg_first - 63 + part * kWave + lane;  // column; key position a - 1
          const bool inside = part * kWave + lane < SEG + kWave && a <= view.len - 1;
          key_in[part] = (inside && a >= 1) ? view.k[a - 1] : 0u;
          old_key_in[part] = (inside && a - W - 2 >= 0) ? view.k[a - W - 2] : 0u;
        }
        const auto store_rows_and_keys = [&]() {
          if (row_lane) {
            uint4* row_words = reinterpret_cast<uint4*>(rows + lane * kRowWords);
            row_words[0] = make_uint4(symbols.x, symbols.z, record.y, record.z);
            row_words[1] = make_uint4(symbols.y, symbols.w, 0u, 0u);
            query_rows[lane] = seg_first + lane < view.steps ? symbols.x : 0u;
          }
#pragma unroll
          for (int part = 0; part < kKeyParts; ++part) {
            if (part * kWave + lane < SEG + kWave) {
              key_window[part * kWave + lane] = key_in[part];
              old_key_window[part * kWave + lane] = old_key_in[part];
            }
          }
        };
        constexpr int kValueParts = ((SEG + kWave) * NVW + kWave - 1) / kWave;
        uint32_t value_in[kValueParts];
#pragma unroll
        for (int part = 0; part < kValueParts; ++part) {
          const int index = part * kWave + lane;
          const int column = index / NVW;
          const int a = seg_first - 63 + column;
          value_in[part] = (want_qk && column < SEG + kWave && a >= 1 && a <= view.len - 1)
              ? view.vbits[static_cast<int64_t>(a) * NVW + (index - column * NVW)] : 0u;
        }
        const auto store_values = [&]() {
          if (want_qk) {
#pragma unroll
            for (int part = 0; part < kValueParts; ++part) {
              if (part * kWave + lane < (SEG + kWave) * NVW) {
                value_window[part * kWave + lane] = value_in[part];
              }
            }
          }
        };
        const auto store_rows_and_columns = [&]() {
          store_rows_and_keys();
          store_values();
        };
        if constexpr (!kFetchAhead) {
          __builtin_amdgcn_sched_barrier(0);
          store_rows_and_columns();
          __builtin_amdgcn_sched_barrier(0);
        }
        constexpr int kGradParts = SEG * kGradChunksMax / kWave;
        static_assert(kGradParts * kWave == SEG * kGradChunksMax, "whole 16-byte pieces per lane");
        // the grad_output rows come in groups that fit the registers free at this point
        constexpr int kGradGroup = kGradParts % 4 == 0 ? 4 : (kGradParts % 3 == 0 ? 3 : 1);
        static_assert(kGradParts % kGradGroup == 0, "whole groups");
        // 16-byte pieces the segment really has (the terms of the input type), numbered row
        // by row: a group of registers then never waits for pieces that do not exist
        const int pieces = SEG * grad_chunks;
        const float per_row = 1.0f / static_cast<float>(grad_chunks);
#pragma unroll
        for (int group = 0; group < kGradParts; group += kGradGroup) {
          if (group * kWave >= pieces) break;  // wave-uniform
          uint4 grad_in[kGradGroup];
#pragma unroll
          for (int part = 0; part < kGradGroup; ++part) {
            const int index = (group + part) * kWave + lane;
            const int r = static_cast<int>((static_cast<float>(index) + 0.5f) * per_row);
            const int piece = index - r * grad_chunks;
            grad_in[part] = make_uint4(0u, 0u, 0u, 0u);
            if (index < pieces && seg_first + r < view.steps) {
              grad_in[part] = *reinterpret_cast<const uint4*>(
                  view.grad_rows +
                  static_cast<int64_t>(view.diag0 + 1 + seg_first + r) * P.grad_pitch + 8 * piece);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (kFetchAhead) {
            if (group == 0) store_rows_and_columns();
          }
#pragma unroll
          for (int part = 0; part < kGradGroup; ++part) {
            const int index = (group + part) * kWave + lane;
            const int r = static_cast<int>((static_cast<float>(index) + 0.5f) * per_row);
            const int piece = index - r * grad_chunks;
            if (index < pieces) {
              *reinterpret_cast<uint4*>(grad_rows_lds + r * GP + 8 * piece) = grad_in[part];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        stage_rows<NVW, kRowFull>(view, seg_first, SEG, lane, rows, W);
        if (lane < SEG) {
          const int i = seg_first + lane;
          query_rows[lane] = i < view.steps ? view.q[view.diag0 + 1 + i] : 0u;
        }
        stage_grad_rows(view, seg_first, SEG, lane, grad_rows_lds, GP, P.grad_pitch);
        for (int index = lane; index < SEG + kWave; index += kWave) {
          const int a = seg_first - 63 + index;  // column; key position a - 1
          key_window[index] = (a >= 1 && a <= view.len - 1) ? view.k[a - 1] : 0u;
          old_key_window[index] = (a - W - 2 >= 0 && a <= view.len - 1) ? view.k[a - W - 2] : 0u;
        }
        if (want_qk) stage_value_columns<NVW>(view, seg_first, SEG + kWave, lane, value_window);
      }
      wave_lds_fence();
      // segment-level forward sweep: checkpoint before every chunk
      const int own_chunks = (seg_last - seg_first + kChunk - 1) / kChunk;
      for (int chunk = 0; !stored && chunk < own_chunks; ++chunk) {
        ck_evidence[chunk * kWave + lane] = band.evidence;
        ck_window[chunk * kWave + lane] = band.window;
        if (chunk + 1 < own_chunks) {
          const int local = chunk * kChunk;
          sweep_rows<NVW, true>(band, rows + local * kRowWords, seg_first + local, kChunk, lane,
                                W, P.gate_log2);
        }
      }
      }  // segment_active

      for (int chunk = chunks - 1; chunk >= 0; --chunk) {
        const int local = chunk * kChunk;               // first row of the chunk inside the segment
        const int first = seg_first + local;            // step index of the chunk's first row
        const int rows_here = min(kChunk, seg_last - first);  // < kChunk only for the band's last rows
        const bool chunk_active = NW == 1 || first < my_steps;
        // rows below the piece: only the reverse recurrences are taken from them
        const bool halo_rows = PIECES && first >= row_end;
        if constexpr (kRecomputeLaneValues) {
          lane = lane_id;
          asm volatile("" : "+v"(lane));
          li = lane & 15;
          lg = lane >> 4;
        }
        if (chunk_active) {
        int window_word;
        uint32_t kept_bits = 0u;  // bit r: row r kept
        if (stored) {
          // this chunk's record arrived while the chunk after it ran; the record of the
          // chunk before it sets out now
          band.evidence = record_evidence;
          window_word = record_window;
          kept_bits = record_kept;
          // the copies are made before the loads set out, so that the loads can land in the
          // record registers (copies after the loads would wait for them)
          asm volatile("" : "+v"(band.evidence), "+v"(window_word), "+v"(kept_bits));
          if (first >= kChunk) fetch_record(first / kChunk - 1);
          __builtin_amdgcn_sched_barrier(0);
        } else {
          // (a use inside this branch: the wait for these loads must not end up behind the
          // branch, where it would also wait for the record loads of the other path)
          float evidence_in = ck_evidence[chunk * kWave + lane];
          int window_in = ck_window[chunk * kWave + lane];
          asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3"
                       : "=&v"(band.evidence), "=&v"(window_word)
                       : "v"(evidence_in), "v"(window_in));
        }
        // stored records say whether any overflow term of the chunk matters
        const bool chunk_quiet =
            stored && (__builtin_amdgcn_readfirstlane(window_word) & 0x8000) == 0;
        band.window = stored ? (window_word & kRecordWindowMax) : window_word;
        // sliding registers of the chunk's first step: column first - lane
        band.key_word = key_window[local + 63 - lane];
        band.old_key_word = old_key_window[local + 63 - lane];
        const uint16_t* grad_tile = grad_rows_lds + local * GP;
        // window column c <-> a = first + 1 - 64 + c (first + 1 is lane 0's column in the first row)
        const uint32_t* key_tile = key_window + local;
        // The one [row][lane] tile holds, in turn, the chunk's utilities, its route
        // weights d*p and its gate adjoints h; each pair's slot is replaced in place.
        if (want_qk) {
          utility_tiles_staged<NVW, DVP, true>(grad_tile, GP, P.grad_pitch / 32,
                                               value_window + local * NVW, sign_table, tile,
                                               kTilePitch, discard, lane);
          wave_lds_fence();
        }
        issue_pending();
        uint32_t route_hash = 0u;
        if constexpr (DROPOUT) {
          if (!stored) route_hash = route_hash_of(first - lane);
        }
        if (!want_qk) {  // no utilities were written: the replay must still read finite values
#pragma unroll
          for (int r = 0; r < kChunk; ++r) tile[r * (kTilePitch + 1) + 64 - lane] = 0.0f;
        }
        float keep_evidence[kChunk];  // S + overflow
        float keep_overflow[kChunk];
        float keep_gate[kChunk];
        float keep_adjoint[kChunk];   // external adjoint A of the route score

        // Forward replay of the chunk, compiled twice: the steady-state form (all
        // lanes past their window fill, full chunk) needs no masking at all.  In
        // the general form rows past the end of the band (only in the band's last
        // chunk) repeat the last row's data and are masked, which keeps the loop
        // free of branches.
        auto replay = [&](auto steady_tag, auto cached_tag, auto quiet_tag) {
          constexpr bool STEADY = decltype(steady_tag)::value;
          constexpr bool CACHED = decltype(cached_tag)::value;  // keep decisions are read back
          constexpr bool QUIET = decltype(quiet_tag)::value;    // overflow terms are negligible
          // (the chunk's offset into the staged rows is held in a vector register: derived
          // from a scalar it was formed again, two instructions, in front of every row's reads)
          uint32_t row_offset = static_cast<uint32_t>(local) * kRowWords;
          asm volatile("" : "+v"(row_offset));
          const uint32_t* row = rows + row_offset;
          const float* slot = tile + 64 - lane;  // this lane's pair of row r: + r * (pitch + 1)
          // row words and utilities are fetched kRowsAhead rows before their use
          constexpr int kRowsAhead = kFetchAhead ? 2 : 1;
          // replay order: everything a quiet chunk reads of a row is one 16-byte word
          constexpr bool kOldWords = !(STEADY && QUIET);
          uint4 ahead_symbols[kRowsAhead];
          uint4 ahead_extra[kRowsAhead];
          float ahead_utility[kRowsAhead];
          const auto fetch_row = [&](int from, int into) {
            ahead_symbols[into] = *reinterpret_cast<const uint4*>(row + from * kRowWords);
            if constexpr (kOldWords) {
              ahead_extra[into] = *reinterpret_cast<const uint4*>(row + from * kRowWords + 4);
            }
            ahead_utility[into] = slot[from * (kTilePitch + 1)];
          };
#pragma unroll
          for (int r = 0; r < kRowsAhead; ++r) fetch_row(r, r);
#pragma unroll
          for (int r = 0; r < kChunk; ++r) {
            const uint4 words = ahead_symbols[r % kRowsAhead];
            uint4 extra = make_uint4(0u, 0u, 0u, 0u);
            if constexpr (kOldWords) extra = ahead_extra[r % kRowsAhead];
            const RowSymbols symbols{words.x, extra.x, words.y, extra.y};
            // the slot holds the pair's utility (anything finite when no symbol
            // gradient is wanted, in which case the adjoint is never used)
            const float utility = ahead_utility[r % kRowsAhead];
            if (r + kRowsAhead < kChunk) fetch_row(r + kRowsAhead, r % kRowsAhead);
            // the loads stay here, ahead of their use (the scheduler would sink them)
            if constexpr (kFetchAhead) __builtin_amdgcn_sched_barrier(0);
            const bool row_ok = r < rows_here;
            const int i = min(first + r, last_step);
            const int t = view.diag0 + 1 + i;
            const float shift = __uint_as_float(words.z);
            const float expected = __uint_as_float(words.w);
            const StepOut s =
                forward_step<NVW, STEADY, QUIET>(band, symbols, i, lane, W, P.gate_log2);
            const float one_plus = 1.0f + s.evidence;
            const float inv_root = fast_rsq(one_plus);
            const float root = one_plus * inv_root;
            const bool live = STEADY || (s.active && row_ok);
            const float probability = live ? fast_exp2(fmaf(root, logit_gain, -shift)) : 0.0f;
            float keep = 1.0f;
            if constexpr (DROPOUT) {
              if constexpr (CACHED) {
                const int kept = __builtin_amdgcn_sbfe(static_cast<int>(kept_bits), r, 1);
                keep = __int_as_float(__float_as_int(inverse_keep) & kept);
              } else {
                route_hash = dpp_wave_shr1(route_hash_of(i + 1), route_hash);
                set_row(key, t);
                keep = dropout_keeps(key, route_hash) ? inverse_keep : 0.0f;
              }
            }
            // (without its constant factor adjoint_gain, which symbol_scale carries)
            const float adjoint = (probability * inv_root) * (keep * utility - expected);
            tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16(probability * keep);
            // rows past the band's end run on repeated data and may hold anything,
            // NaN included: select, never multiply by zero
            keep_adjoint[r] = live ? adjoint : 0.0f;
            keep_gate[r] = live ? s.gate : 0.0f;
            keep_overflow[r] = live ? s.overflow : 0.0f;
            keep_evidence[r] = live ? (QUIET ? s.evidence : s.evidence + s.overflow) : 0.0f;
          }
        };
        const bool steady = first >= W + kWave && rows_here == kChunk;
        // A quiet chunk takes no overflow term and tracks no window, so its unmasked form
        // only needs every lane to have a pair in every row: from the band's row 64 on, not
        // only once the windows are full.
        const bool unmasked_quiet = chunk_quiet && first >= kWave && rows_here == kChunk;
        const bool cached = DROPOUT && stored;
        if (unmasked_quiet) {
          if (cached) replay(std::true_type{}, std::true_type{}, std::true_type{});
          else replay(std::true_type{}, std::false_type{}, std::true_type{});
        } else if (steady) {
          if (cached) replay(std::true_type{}, std::true_type{}, std::false_type{});
          else replay(std::true_type{}, std::false_type{}, std::false_type{});
        } else {
          if (cached) replay(std::false_type{}, std::true_type{}, std::false_type{});
          else replay(std::false_type{}, std::false_type{}, std::false_type{});
        }
        wave_lds_fence();

        // Column sums.  Tile m covers window columns 16m .. 16m+15 (a = first + 1 - 64 + c);
        // element (column c, row r) of the matrix is tile[r][c], a dword
        // holding the two bfloat16 terms of the pair's value.  One matrix instruction per
        // tile contracts all 16 rows: k = 2 r + term, lane (li, lg) brings rows 4 lg .. 4 lg + 3
        // of column 16 m + li.
        const auto column_operands = [&](v4u (&operands)[kWindowTiles]) {
#pragma unroll
          for (int m = 0; m < kWindowTiles; ++m) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int r = 4 * lg + j;
              operands[m][j] = tile_bits[r * kTilePitch + 16 * m + li];
            }
          }
        };
        if (want_v && !halo_rows) {
          // the other factor: grad_output of the same rows, term by term, each element
          // repeated for the two terms of the weight (the third term of a float32
          // grad_output is below the accuracy of the split weights and is left out).
          // Where registers allow, every LDS read of the section is issued before the first
          // is used: one latency instead of one per operand.
          const int terms = P.grad_terms < 2 ? P.grad_terms : 2;
          constexpr bool kReadsFirst = VT <= 2;
          uint32_t elements[VT][2][4];
          if constexpr (kReadsFirst) {
#pragma unroll
            for (int n = 0; n < VT; ++n) {
              const int d = 16 * n + li;
              const uint16_t* source = grad_tile + (4 * lg) * GP + (d < DVP ? d : DVP - 1);
#pragma unroll
              for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  // a second term that does not exist is read from the first and not used
                  elements[n][t][j] = source[j * GP + (t < terms ? t : 0) * DVP];
                }
              }
            }
          }
          v4u weights[kWindowTiles];
          column_operands(weights);
          if constexpr (kReadsFirst) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int n = 0; n < VT; ++n) {
            const int d = 16 * n + li;
            const uint16_t* source = grad_tile + (4 * lg) * GP + (d < DVP ? d : DVP - 1);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              if (t >= terms) break;  // wave-uniform
              v4u grads;
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const uint32_t element =
                    kReadsFirst ? elements[n][t][j] : uint32_t(source[j * GP + t * DVP]);
                grads[j] = d < DVP ? element | (element << 16) : 0u;
              }
#pragma unroll
              for (int m = 0; m < kWindowTiles; ++m) {
                value_acc[m][n] = mfma_bf16(weights[m], grads, value_acc[m][n]);
              }
            }
          }
        }

        if (want_qk) {
          wave_lds_fence();
          // reverse walk of the chunk: gate adjoints replace the weights
          const bool quiet = unmasked_quiet && ring_live == 0;
          if (quiet) {
            // no overflow term of the chunk can move a gradient and the ring is empty:
            // h = b (S + o), nothing to mask
#pragma unroll
            for (int r = kChunk - 1; r >= 0; --r) {
              float b;
              if constexpr (TERMS == 2) {
                b = fmaf(gate_below, adjoint_carry, keep_adjoint[r]);
              } else {
                b = carry_step(gate_below, adjoint_carry, keep_adjoint[r], carry_rest);
              }
              adjoint_carry = b;
              gate_below = keep_gate[r];
              if constexpr (TERMS == 2) {
                tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16(b * keep_evidence[r]);
              } else {
                uint32_t rest;
                tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16_exact(
                    fmaf(b, keep_evidence[r], carry_rest * keep_evidence[r]), rest);
                rest_plane[r * (kRestPitch + 1) + 64 - lane] = static_cast<uint16_t>(rest >> 16);
              }
            }
          } else {
#pragma unroll
          for (int r = kChunk - 1; r >= 0; --r) {
            const int i = first + r;
            float b;
            if constexpr (TERMS == 2) {
              b = fmaf(gate_below, adjoint_carry, keep_adjoint[r]);
            } else {
              b = carry_step(gate_below, adjoint_carry, keep_adjoint[r], carry_rest);
            }
            adjoint_carry = b;
            gate_below = keep_gate[r];
            const float overflow = keep_overflow[r];
            const float term = overflow >= P.tail_threshold ? b * overflow : 0.0f;
            [[maybe_unused]] float term_low = 0.0f;
            if constexpr (TERMS == 3) {
              term_low = overflow >= P.tail_threshold
                  ? fmaf(carry_rest, overflow, fmaf(b, overflow, -term)) : 0.0f;
            }
            const bool any_term = __ballot(term != 0.0f) != 0ull;
            if (any_term) {
              if (ring_live == 0) ring_fresh = P.ring_rows;
              ring_live = P.ring_rows;
            }
            if (ring_live > 0) {
              const int slot = i % P.ring_rows;
              float leaving = 0.0f;
              [[maybe_unused]] float leaving_low = 0.0f;
              if (ring_fresh > 0) {
                --ring_fresh;
              } else {
                leaving = ring[slot * kWave + lane];
                if constexpr (TERMS == 3) {
                  leaving_low = __uint_as_float(uint32_t(ring_low[slot * kWave + lane]) << 16);
                }
              }
              ring[slot * kWave + lane] = term;
              if constexpr (TERMS == 2) {
                ring_sum += term - leaving;
              } else {
                // the low part enters the sum as it is stored, so that it leaves as it entered
                const uint32_t low_bits = __float_as_uint(term_low) & 0xffff0000u;
                ring_low[slot * kWave + lane] = static_cast<uint16_t>(low_bits >> 16);
                const float added = __fadd_rn(ring_sum, term);
                const float added_rest = __fsub_rn(term, __fsub_rn(added, ring_sum));
                const float left = __fsub_rn(added, leaving);
                const float left_rest = __fsub_rn(__fsub_rn(added, left), leaving);
                ring_sum = left;
                ring_sum_low += (__uint_as_float(low_bits) - leaving_low) + (added_rest + left_rest);
              }
              --ring_live;
            }
            const float h = TERMS == 2
                ? fmaf(b, keep_evidence[r], -ring_sum)
                : fmaf(b, keep_evidence[r], -ring_sum) +
                      fmaf(carry_rest, keep_evidence[r], -ring_sum_low);
            if (ring_live == 0) {
              ring_sum = 0.0f;
              if constexpr (TERMS == 3) ring_sum_low = 0.0f;
            }
            const bool active = steady || ((i + 1 - lane) >= 1 && r < rows_here);
            if constexpr (TERMS == 2) {
              tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16(active ? h : 0.0f);
            } else {
              uint32_t rest;
              tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16_exact(active ? h : 0.0f, rest);
              rest_plane[r * (kRestPitch + 1) + 64 - lane] = static_cast<uint16_t>(rest >> 16);
            }
          }
          }
          wave_lds_fence();

          if (want_k && !halo_rows) {
            v4u adjoints[kWindowTiles];
            v2u adjoint_rests[kWindowTiles];  // the third terms: k = r, a product of their own
            column_operands(adjoints);
#pragma unroll
            for (int m = 0; m < kWindowTiles; ++m) {
              if constexpr (TERMS == 2) break;
              const uint16_t* column = rest_plane + 16 * m + li;
              const int r = 4 * lg;
              adjoint_rests[m] = v2u{
                  pair_of(column + r * kRestPitch, column + (r + 1) * kRestPitch),
                  pair_of(column + (r + 2) * kRestPitch, column + (r + 3) * kRestPitch)};
            }
            const uint4 q_words = *reinterpret_cast<const uint4*>(query_rows + local + 4 * lg);
#pragma unroll
            for (int n = 0; n < DT; ++n) {
              const int bit = 16 * n + li;
              const v4u symbols = {negated_symbol_pair(q_words.x, bit), negated_symbol_pair(q_words.y, bit),
                                   negated_symbol_pair(q_words.z, bit), negated_symbol_pair(q_words.w, bit)};
              // one element per row for the third terms: low half of one row, high half of the next
              const v2u symbols_once = {__builtin_amdgcn_perm(symbols[1], symbols[0], 0x07060100u),
                                        __builtin_amdgcn_perm(symbols[3], symbols[2], 0x07060100u)};
              // A 16x16x16 product that accumulates onto the result of a 16x16x32 product
              // must not issue right behind it: the compiler leaves out the wait states
              // this pair needs (seen as wrong sums), so the two shapes run as separate
              // groups with the wait states written out between them.
#pragma unroll
              for (int m = 0; m < kWindowTiles; ++m) {
                key_acc[m][n] = mfma_bf16(adjoints[m], symbols, key_acc[m][n]);
              }
              if constexpr (TERMS == 3) {
                mfma_shape_change();
#pragma unroll
                for (int m = 0; m < kWindowTiles; ++m) {
                  key_acc[m][n] = mfma_bf16_k16(adjoint_rests[m], symbols_once, key_acc[m][n]);
                }
                mfma_shape_change();
              }
            }
          }
          // row sums: rows are complete for this band after the chunk
          if (want_q && !halo_rows) {
            // k slice lg of step s <-> window columns 20 lg + 4 s .. + 3 (both terms of each):
            // every lane reads 20 consecutive key words and 20 consecutive columns of its row
            // the third terms accumulate apart (see above: one instruction shape per
            // accumulator chain)
            v4f query_part[3][DT];
#pragma unroll
            for (int part = 0; part < 3; ++part) {
#pragma unroll
              for (int n = 0; n < DT; ++n) query_part[part][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            }
            // Where registers allow, every LDS read of the section is issued before the first
            // product (one latency instead of one per step); the widest tile reads step by step.
            constexpr bool kReadsFirst = VT <= 2;
            constexpr int kHeld = kReadsFirst ? kWindowTiles : 1;
            uint4 k_words_of[kHeld];
            v4u adjoints_of[kHeld];
            v2u adjoint_rests_of[kHeld];
            const auto read_step = [&](int step, int slot) {
              // four neighbouring columns of row li: one aligned 16-byte word of the tile and
              // one aligned 8-byte word of the third terms
              const int c0 = 4 * kWindowTiles * lg + 4 * step;
              k_words_of[slot] = *reinterpret_cast<const uint4*>(key_tile + c0);
              adjoints_of[slot] = *reinterpret_cast<const v4u*>(tile_bits + li * kTilePitch + c0);
              if constexpr (TERMS == 3) {
                adjoint_rests_of[slot] =
                    *reinterpret_cast<const v2u*>(rest_plane + li * kRestPitch + c0);
              }
            };
            if constexpr (kReadsFirst) {
#pragma unroll
              for (int step = 0; step < kWindowTiles; ++step) read_step(step, step);
              __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int step = 0; step < kWindowTiles; ++step) {
              if constexpr (!kReadsFirst) read_step(step, 0);
              const uint4 k_words = k_words_of[kReadsFirst ? step : 0];
              const v4u adjoints = adjoints_of[kReadsFirst ? step : 0];
              const v2u adjoint_rests = adjoint_rests_of[kReadsFirst ? step : 0];
#pragma unroll
              for (int n = 0; n < DT; ++n) {
                const int bit = 16 * n + li;
                const v4u symbols = {negated_symbol_pair(k_words.x, bit), negated_symbol_pair(k_words.y, bit),
                                     negated_symbol_pair(k_words.z, bit), negated_symbol_pair(k_words.w, bit)};
                const v2u symbols_once = {__builtin_amdgcn_perm(symbols[1], symbols[0], 0x07060100u),
                                          __builtin_amdgcn_perm(symbols[3], symbols[2], 0x07060100u)};
                query_part[step & 1][n] = mfma_bf16(adjoints, symbols, query_part[step & 1][n]);
                if constexpr (TERMS == 3) {
                  query_part[2][n] = mfma_bf16_k16(adjoint_rests, symbols_once, query_part[2][n]);
                }
              }
            }
#pragma unroll
            for (int n = 0; n < DT; ++n) {
              done_query[n] = (query_part[0][n] + query_part[1][n]) + query_part[2][n];
            }
          }
        }
        // the last window tile (columns first + 1 .. first + 16) is complete: park it with
        // the chunk's row sums, then shift the window up by one tile
        if (!halo_rows) {
#pragma unroll
        for (int n = 0; n < VT; ++n) done_value[n] = value_acc[kWindowTiles - 1][n];
#pragma unroll
        for (int n = 0; n < DT; ++n) done_key[n] = key_acc[kWindowTiles - 1][n];
        done_first = first;
        done_rows = rows_here;
#pragma unroll
        for (int m = kWindowTiles - 1; m > 0; --m) {
#pragma unroll
          for (int n = 0; n < VT; ++n) value_acc[m][n] = value_acc[m - 1][n];
#pragma unroll
          for (int n = 0; n < DT; ++n) key_acc[m][n] = key_acc[m - 1][n];
        }
#pragma unroll
        for (int n = 0; n < VT; ++n) value_acc[0][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int n = 0; n < DT; ++n) key_acc[0][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }  // !halo_rows
        wave_lds_fence();
        }  // chunk_active

        if constexpr (NW > 1) {
          // Every band of the block has just completed the same 16 columns (same band-local
          // step) and, of its rows, a tile that the next band meets four chunks from now.
          const int g = first / kChunk;
          const int tile_floats = P.exchange_tile_floats;
          // a tile in LDS: 16 bytes per lane, only the lanes of columns 0 .. 7 when narrow
          const bool narrow_tiles = tile_floats == exchange_tile_floats(true);
          const bool tile_lane = !narrow_tiles || li < 8;
          const int tile_offset = narrow_tiles ? 4 * (8 * lg + (li & 7)) : 4 * lane;
          if (chunk_active) {
            // both waves have this chunk: each takes over one kind of column sums
            const bool both = first < lead_steps - kWave;
            done_flush_value = wave == 0;
            done_flush_key = wave == 1 || !both;
            done_flush_rows = true;
            if (row_queue_on && want_q) {
              if (wave == 1 && tile_lane) {  // what band 0 summed over these rows, four chunks ago
                const float* slot = row_queue + ((g % kQueueSlots) * DT) * tile_floats + tile_offset;
#pragma unroll
                for (int n = 0; n < DT; ++n) {
                  done_query[n] += *reinterpret_cast<const v4f*>(slot + n * tile_floats);
                }
              }
              // Rows above the first row of band 1 (chunks 0 .. 3 of band 0) and the rows of
              // band 1 go to memory from here; the others wait in the queue for band 1.
              if (wave == 0 && g >= 4 && lead_steps - kWave > 0) done_flush_rows = false;
            }
            // value tiles of wave 1 go to wave 0, key tiles of wave 0 to wave 1
            if (both && tile_lane) {
              float* out = column_exchange + tile_offset;
              if (wave == 1 && want_v) {
#pragma unroll
                for (int n = 0; n < VT; ++n) {
                  *reinterpret_cast<v4f*>(out + n * tile_floats) = done_value[n];
                }
              }
              if (wave == 0 && want_k) {
#pragma unroll
                for (int n = 0; n < DT; ++n) {
                  *reinterpret_cast<v4f*>(out + (VT + n) * tile_floats) = done_key[n];
                }
              }
            }
          }
          block_barrier();
          if (row_queue_on && want_q && wave == 0 && chunk_active && !done_flush_rows && tile_lane) {
            // band 1 has taken the slot's old tile in front of the barrier
            float* slot = row_queue + ((g % kQueueSlots) * DT) * tile_floats + tile_offset;
#pragma unroll
            for (int n = 0; n < DT; ++n) {
              *reinterpret_cast<v4f*>(slot + n * tile_floats) = done_query[n];
            }
          }
          if (chunk_active && tile_lane && first < lead_steps - kWave) {
            const float* in = column_exchange + tile_offset;
            if (wave == 0 && want_v) {
#pragma unroll
              for (int n = 0; n < VT; ++n) {
                done_value[n] += *reinterpret_cast<const v4f*>(in + n * tile_floats);
              }
            }
            if (wave == 1 && want_k) {
#pragma unroll
              for (int n = 0; n < DT; ++n) {
                done_key[n] += *reinterpret_cast<const v4f*>(in + (VT + n) * tile_floats);
              }
            }
          }
          // the column tiles have been taken over: the waves may store their next ones
          block_barrier();
        }
        // wide tiles have no registers to spare for carrying the results across a chunk
        if constexpr (kFlushAtOnce) {
          if (chunk_active) {
            // The record of the next chunk has been on its way for a whole chunk: it is
            // taken in now, so that the next chunk does not wait for it behind the atomics
            // issued here (memory operations of a wave are counted in order).
            if (stored) {
              asm volatile("" : : "v"(record_evidence), "v"(record_window), "v"(record_kept));
            }
            issue_pending();
          }
        }
      }
    }
    issue_pending();
    if (PIECES && row_begin > 0) {
      // A piece that does not start its band leaves partial sums of the 64 columns to the left
      // of its first row's column; the piece above adds the rest.  After the last shift tile m
      // holds columns row_begin - 79 + 16 m .. + 15, i.e. it is the tile a chunk starting at
      // row row_begin - 80 + 16 m would have completed.
      done_has_rows = false;
#pragma unroll
      for (int m = 1; m < kWindowTiles; ++m) {
#pragma unroll
        for (int n = 0; n < VT; ++n) done_value[n] = value_acc[m][n];
#pragma unroll
        for (int n = 0; n < DT; ++n) done_key[n] = key_acc[m][n];
        done_first = row_begin - 16 * kWindowTiles + 16 * m;
        done_rows = kChunk;
        issue_pending();
      }
    }
  }
}

// Slots of a tile family's table of kernel addresses (rosa_vjp_instances.hip fills it,
// rosa_kernels.hip launches from it).
constexpr int kGradientFormOneWave = 0;   // single-wave blocks, whole bands
constexpr int kGradientFormTwoWaves = 1;  // two-wave blocks
constexpr int kGradientFormPieces = 2;    // single-wave blocks, bands cut into pieces
constexpr int vjp_kernel_slot_row_max(int varlen) { return varlen; }
constexpr int vjp_kernel_slot_row_stats(int varlen, int dropout) { return 2 + 2 * varlen + dropout; }
constexpr int vjp_kernel_slot_gradients(int varlen, int dropout, int form, int terms) {
  return 6 + ((2 * varlen + dropout) * 3 + form) * 2 + (terms - 2);
}
constexpr int kVjpKernelSlots = 6 + 4 * 3 * 2;

}  // namespace
