// Device helpers and the problem layout shared by every translation unit of the library
// (see rosa_kernels.hip for the work decomposition).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <type_traits>

#include "../../include/rosa_soft_hip.h"

namespace {

constexpr int kWave = 64;
constexpr float kNullScore = 0.5f;
constexpr float kSqrtScale = 2.414213562373095f;  // sqrt(2) + 1
constexpr float kLog2e = 1.4426950408889634f;

constexpr int kChunk = 16;     // rows kept in registers between the forward and reverse sweeps

// ---------------------------------------------------------------------------
// small device helpers
// ---------------------------------------------------------------------------

__device__ __forceinline__ int dpp_wave_shr1(int fill_lane0, int src) {
  // lane i receives src of lane i-1; lane 0 receives fill_lane0
  return __builtin_amdgcn_update_dpp(fill_lane0, src, 0x138, 0xf, 0xf, false);
}

__device__ __forceinline__ uint32_t dpp_wave_shr1(uint32_t fill_lane0, uint32_t src) {
  return static_cast<uint32_t>(
      dpp_wave_shr1(static_cast<int>(fill_lane0), static_cast<int>(src)));
}

// lanes 8..15 of every 16 receive src of the lane eight below; lanes 0..7 keep `keep`
__device__ __forceinline__ float dpp_row_shr8(float keep, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(keep), __float_as_int(src),
                                                    0x118, 0xf, 0xf, false));
}

// The band kernels run one wavefront per block (or waves that meet at barriers of their
// own).  LDS instructions of one wave execute in order, so data written by one lane is
// visible to another lane's later read without a barrier and without a wait; what is needed
// is that the compiler keeps the order of the accesses, and nothing else: a
// __syncthreads() would also wait for every outstanding global store and atomic, and an
// s_waitcnt here would expose an LDS round trip at every phase of a chunk.
__device__ __forceinline__ void wave_lds_fence() {
  asm volatile("" ::: "memory");
}

// Meeting point of the waves of a block that exchange data through LDS only: the LDS
// traffic of the wave is complete, global stores and atomics stay in flight.
__device__ __forceinline__ void block_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_max(float acc, float src) {
  // lanes without a valid source keep their own value
  const int moved = __builtin_amdgcn_update_dpp(
      __float_as_int(acc), __float_as_int(src), CTRL, ROW_MASK, 0xf, false);
  return fmaxf(acc, __int_as_float(moved));
}

// Maximum over the 64 lanes; the result is valid in lane 63 only.
__device__ __forceinline__ float wave_max_lane63(float v) {
  v = dpp_max<0x111, 0xf>(v, v);
  v = dpp_max<0x112, 0xf>(v, v);
  v = dpp_max<0x114, 0xf>(v, v);
  v = dpp_max<0x118, 0xf>(v, v);
  v = dpp_max<0x142, 0xa>(v, v);
  v = dpp_max<0x143, 0xc>(v, v);
  return v;
}

// A wave-uniform value as a vector register.  Simple vector instructions (add, multiply,
// fma, logic, right shifts) issue at twice the rate of the others on gfx950 when two waves
// share a SIMD, but not when one of their operands is a scalar register: constants of the
// innermost loops are therefore copied once.
__device__ __forceinline__ float in_vector_register(float uniform) {
  float copy;
  asm volatile("v_mov_b32 %0, %1" : "=v"(copy) : "s"(uniform));
  return copy;
}

__device__ __forceinline__ uint32_t in_vector_register(uint32_t uniform) {
  uint32_t copy;
  asm volatile("v_mov_b32 %0, %1" : "=v"(copy) : "s"(uniform));
  return copy;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rsq(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float fast_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }

// popcount(x) + addend in the one instruction the hardware has for it.  (Written out because
// the compiler turns an addend whose set bits lie above the count into an `or` and then no
// longer finds the instruction's own addend.)
__device__ __forceinline__ uint32_t popc_plus(uint32_t x, uint32_t addend) {
  uint32_t result;
  asm("v_bcnt_u32_b32 %0, %1, %2" : "=v"(result) : "v"(x), "v"(addend));
  return result;
}

template <int DTYPE>
__device__ __forceinline__ float load_as_float(const void* base, int64_t index) {
  if constexpr (DTYPE == ROSA_DTYPE_F32) {
    return static_cast<const float*>(base)[index];
  } else if constexpr (DTYPE == ROSA_DTYPE_F16) {
    return static_cast<float>(static_cast<const _Float16*>(base)[index]);
  } else {
    const uint32_t bits = static_cast<const uint16_t*>(base)[index];
    return __uint_as_float(bits << 16);
  }
}

template <int DTYPE>
__device__ __forceinline__ void store_sign(void* base, int64_t index, int sign) {
  // sign in {-1, 0, +1}
  if constexpr (DTYPE == ROSA_DTYPE_F32) {
    static_cast<float*>(base)[index] = static_cast<float>(sign);
  } else if constexpr (DTYPE == ROSA_DTYPE_F16) {
    static_cast<uint16_t*>(base)[index] =
        sign == 0 ? uint16_t(0) : (sign > 0 ? uint16_t(0x3C00) : uint16_t(0xBC00));
  } else {
    static_cast<uint16_t*>(base)[index] =
        sign == 0 ? uint16_t(0) : (sign > 0 ? uint16_t(0x3F80) : uint16_t(0xBF80));
  }
}

template <int DTYPE>
__device__ __forceinline__ void store_nan(void* base, int64_t index) {
  if constexpr (DTYPE == ROSA_DTYPE_F32) {
    static_cast<uint32_t*>(base)[index] = 0x7fc00000u;
  } else if constexpr (DTYPE == ROSA_DTYPE_F16) {
    static_cast<uint16_t*>(base)[index] = uint16_t(0x7e00);
  } else {
    static_cast<uint16_t*>(base)[index] = uint16_t(0x7fc0);
  }
}

// The counter hash (reference rosa_soft_kernels.cu:549-586) is six rounds of
//   h(x): x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16
// chained as s = h(s ^ key).  fold16(x) = x ^ (x >> 16) is linear over xor and its own
// inverse, so the closing fold of one round, the key and the opening fold of the next
// round collapse into one xor:  fold16(fold16(x) ^ key) = x ^ fold16(key).  The rounds
// below therefore carry the state *before* its closing fold and take keys that are
// already folded; only the last round is closed.  Same bits, two instructions fewer per
// round.  (The two 32-bit multiplies are slow instructions; building them from 16-bit
// dot products, v_dot2_u32_u16, was measured slower on gfx950.)
__device__ __forceinline__ uint32_t fold16(uint32_t x) { return x ^ (x >> 16); }

__device__ __forceinline__ uint32_t open_round(uint32_t folded_input) {
  uint32_t s = folded_input * 0x7feb352du;
  s ^= s >> 15;
  return s * 0x846ca68bu;
}

// Wave-uniform part of the dropout decision of one (row, route): the folded keys of
// rounds two to six and the integer form of the keep test.
struct DropoutKey {
  uint32_t row_key;    // fold16(row ^ 0xb5297a4d)
  uint32_t head_key;   // fold16(head ^ 0x63d83595)
  uint32_t batch_key;  // fold16(batch ^ 0xa511e9b3)
  uint32_t seed_low_key;
  uint32_t seed_high_key;  // fold16(seed_high ^ 0x9e3779b9)
  uint32_t keep_from;      // keep iff the hash is at least this
};

// The uniform of a pair is (hash >> 8) * 2^-24 and the pair is kept iff uniform >= p.
// Both sides are exact in float32, so this is hash >= ceil(p * 2^24) * 256.
__device__ __forceinline__ DropoutKey make_dropout_key(uint64_t seed, int head, int batch,
                                                       float dropout_p) {
  DropoutKey key;
  key.row_key = 0;
  key.head_key = fold16(static_cast<uint32_t>(head) ^ 0x63d83595u);
  key.batch_key = fold16(static_cast<uint32_t>(batch) ^ 0xa511e9b3u);
  key.seed_low_key = fold16(static_cast<uint32_t>(seed));
  key.seed_high_key = fold16(static_cast<uint32_t>(seed >> 32) ^ 0x9e3779b9u);
  key.keep_from = static_cast<uint32_t>(ceilf(dropout_p * 16777216.0f)) << 8;
  return key;
}

__device__ __forceinline__ void set_row(DropoutKey& key, int row) {
  key.row_key = fold16(static_cast<uint32_t>(row) ^ 0xb5297a4du);
}

// first hash round (open): depends on the route only, so a band computes it once per
// column (for the column entering at lane 0) and slides it with the columns
__device__ __forceinline__ uint32_t route_hash_of(int route) {
  return open_round(fold16(static_cast<uint32_t>(route) ^ 0x68e31da4u));
}

__device__ __forceinline__ bool dropout_keeps(const DropoutKey& key, uint32_t route_hash) {
  uint32_t s = open_round(route_hash ^ key.row_key);
  s = open_round(s ^ key.head_key);
  s = open_round(s ^ key.batch_key);
  s = open_round(s ^ key.seed_low_key);
  s = open_round(s ^ key.seed_high_key);
  return fold16(s) >= key.keep_from;
}

// ---------------------------------------------------------------------------
// layout
// ---------------------------------------------------------------------------

struct Layout {
  int B, T, N, S, H, D, Hv, Dv, W;
  int varlen;
  // packed-sequence tables (device), valid when varlen != 0
  const int32_t* seq_start;
  const int32_t* seq_len;
  const int32_t* block_prefix;  // [S+1] prefix sums of ceil(len / 64)
  const int64_t* step_prefix;   // [S+1] prefix sums of band_steps_total(len)
  int slots;                    // number of 64-row block slots over all sequences (upper bound)
};

// number of (row, band) steps of one (sequence, head) of length `len`, and the
// number that precede band j: the index space of the chunk records
__host__ __device__ inline int64_t band_steps_total(int len) {
  if (len < 2) return 0;
  const int64_t bands = (len - 2) / 64 + 1;
  return bands * (len - 1) - 32 * bands * (bands - 1);
}

__host__ __device__ inline int64_t band_steps_before(int len, int band) {
  return static_cast<int64_t>(band) * (len - 1) - 32 * static_cast<int64_t>(band) * (band - 1);
}

// The row-statistics pass leaves a record per 16-row chunk of a band for the gradient
// pass, 64 lanes each: S of every diagonal before the chunk's first row (float), the window
// count there as 16 bits (saturated at kRecordWindowMax; bit 15 is set, in every lane, when
// some overflow term of the chunk is large enough to matter) and, with dropout, the keep
// decisions of the chunk (bit r of lane l's 16-bit word = row r, diagonal l): 0.375 bytes
// per pair, 0.5 with dropout.  A saturated count is exact where it matters: the launch keeps
// records only when every count that can still produce a relevant overflow term within a
// chunk lies below the saturation value.
// Chunk c of the band with global step offset `steps_before` and global band number
// `bands_before` owns slot steps_before / 16 + bands_before + c (distinct for all
// chunks of all bands, because a band of n steps has fewer than n / 16 + 2 chunks).
constexpr int kRecordWindowMax = 0x7fff;
constexpr int kCheckpointFloats = 96;   // S [64 lanes], then the 16-bit window words
constexpr int kKeepBitFloats = 32;      // 64 lanes x 16 bits
__host__ __device__ inline int64_t checkpoint_slots(int64_t steps, int64_t bands) {
  return steps / 16 + bands + 1;
}

struct Unit {
  int seq;     // batch index (dense) or packed sequence index
  int block;   // 64-row block / 64-diagonal band index inside the sequence
  int start;   // first token of the sequence in token-major tensors
  int len;     // sequence length
  int head;
  int64_t word_base;  // offset of (seq, head, t = 0) in the head-major word tensors
  bool valid;
};

// slot order is block-major so that equal block indices of all sequences are adjacent
template <bool VARLEN>
__device__ __forceinline__ Unit decode_unit(const Layout& L, int unit_index) {
  Unit u;
  u.head = unit_index % L.H;
  const int slot = unit_index / L.H;
  u.valid = true;
  if constexpr (VARLEN) {
    int low = 0, high = L.S;  // find seq with prefix[seq] <= slot < prefix[seq+1]
    while (low < high) {
      const int mid = (low + high) >> 1;
      if (L.block_prefix[mid + 1] <= slot) low = mid + 1; else high = mid;
    }
    if (low >= L.S) {
      u.valid = false;
      u.seq = 0; u.block = 0; u.start = 0; u.len = 0; u.word_base = 0;
      return u;
    }
    u.seq = low;
    u.block = slot - L.block_prefix[low];
    u.start = L.seq_start[low];
    u.len = L.seq_len[low];
    u.word_base = static_cast<int64_t>(u.head) * L.N + u.start;
  } else {
    u.seq = slot % L.B;
    u.block = slot / L.B;
    u.start = u.seq * L.T;
    u.len = L.T;
    u.word_base = (static_cast<int64_t>(u.seq) * L.H + u.head) * L.T;
  }
  return u;
}

}  // namespace
