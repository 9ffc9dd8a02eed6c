// MI355X (gfx950, wave64) kernels and C ABI of the rosa_soft training operators.
//
// Work decomposition
// ------------------
// A (row t, route a) pair compares the query suffix ending at t with the key
// suffix ending at a-1.  Every recurrence of the operator runs along a
// diagonal t - a = const, so the pair space of one (sequence, head) is cut
// into BANDS of 64 adjacent diagonals.  One wavefront owns one band; lane l
// owns diagonal 64*j + l and the wave marches over rows t, so that at a given
// step every lane works on the same row t (row data is wave-uniform and lives
// in scalar registers) while the per-column data (key word, value sign bits)
// slides from lane to lane with one DPP wave shift per step.  All suffix
// state (run length, soft evidence, window mismatch count, reverse adjoint)
// is private to a lane: no cross-lane traffic is needed for the recurrences.
//
// The hard forward uses the transposed arrangement (lane = row, the wave walks
// over routes) because its only reduction is per row.
//
// Numerics: every score, normaliser and gradient is float32; exp/rsqrt use the
// hardware approximations, like the reference's --use_fast_math build.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <type_traits>

#include "../../include/rosa_soft_hip.h"

#include <mutex>

// Scratch memory of rosa_hip_hard_forward_static: the forward's workspace (route of every
// row and the packed-sequence tables) for callers that cannot allocate.  Every device the
// library runs on holds its own copy until the process ends.  In host code the array's name
// is not a device address: the address of a device's copy comes from hipGetSymbolAddress.
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kWave = 64;
constexpr float kNullScore = 0.5f;
constexpr float kSqrtScale = 2.414213562373095f;  // sqrt(2) + 1
constexpr float kLog2e = 1.4426950408889634f;

constexpr int kChunk = 16;     // rows kept in registers between the forward and reverse sweeps

thread_local char g_error[512] = "";

int fail(int code, const char* message) {
  snprintf(g_error, sizeof(g_error), "%s", message);
  return code;
}

int fail_hip(hipError_t status, const char* what) {
  snprintf(g_error, sizeof(g_error), "%s: %s", what, hipGetErrorString(status));
  return 100 + static_cast<int>(status);
}

// Optional stage timing: when enabled, every launch sequence brackets its
// stages with HIP events recorded on the caller's stream.  Nothing is read
// back until rosa_hip_stage_times() is called.
enum Stage { kStageForward = 0, kStagePrepare, kStageRowMax, kStageRowStats, kStageGradients,
             kStageFinalize, kStageCount };

struct StageTimer {
  bool enabled = false;
  bool created = false;
  hipEvent_t begin[kStageCount];
  hipEvent_t end[kStageCount];
  bool used[kStageCount];
};

StageTimer g_timer;

void stage_begin(Stage stage, hipStream_t stream) {
  if (!g_timer.enabled) return;
  g_timer.used[stage] = true;
  (void)hipEventRecord(g_timer.begin[stage], stream);
}

void stage_end(Stage stage, hipStream_t stream) {
  if (!g_timer.enabled) return;
  (void)hipEventRecord(g_timer.end[stage], stream);
}

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

// ---------------------------------------------------------------------------
// packed-sequence table: sanitised offsets and block prefix sums
// ---------------------------------------------------------------------------

__global__ void prepare_sequences_kernel(const int32_t* __restrict__ cu_seqlens, int S, int N,
                                         int32_t* __restrict__ seq_start,
                                         int32_t* __restrict__ seq_len,
                                         int32_t* __restrict__ block_prefix,
                                         int64_t* __restrict__ step_prefix, int H,
                                         int64_t checkpoint_capacity,
                                         int32_t* __restrict__ header) {
  // Single block.  Offsets are valid iff they start at 0, end at N and never decrease.
  // When they are not, every sequence is made empty, so that no later kernel touches a
  // token, and header[0] is set: the kernels that write results then fill them with NaN.
  __shared__ int bad;
  __shared__ int partial[256];
  if (threadIdx.x == 0) bad = (cu_seqlens[0] != 0 || cu_seqlens[S] != N) ? 1 : 0;
  __syncthreads();
  const int per_thread = (S + blockDim.x - 1) / blockDim.x;
  const int first = threadIdx.x * per_thread;
  const int last = min(S, first + per_thread);
  int local_bad = 0;
  for (int s = first; s < last; ++s) {
    if (cu_seqlens[s] > cu_seqlens[s + 1]) local_bad = 1;
  }
  if (local_bad) atomicOr(&bad, 1);
  __syncthreads();
  const bool valid = bad == 0;
  int blocks = 0;
  for (int s = first; s < last; ++s) {
    const int begin = valid ? cu_seqlens[s] : 0;
    const int length = valid ? cu_seqlens[s + 1] - begin : 0;
    seq_start[s] = begin;
    seq_len[s] = length;
    blocks += (length + 63) >> 6;
  }
  partial[threadIdx.x] = blocks;
  __syncthreads();
  if (threadIdx.x == 0) {
    int running = 0;
    for (int i = 0; i < static_cast<int>(blockDim.x); ++i) {
      const int value = partial[i];
      partial[i] = running;
      running += value;
    }
    block_prefix[S] = running;
    header[0] = bad;
  }
  __syncthreads();
  if (threadIdx.x == 0 && step_prefix != nullptr) {
    // index space of the chunk records; they are used only if they fit
    int64_t steps = 0;
    for (int s = 0; s < S; ++s) {
      step_prefix[s] = steps;
      steps += band_steps_total(seq_len[s]);
    }
    step_prefix[S] = steps;
    header[3] = checkpoint_slots(steps * H, static_cast<int64_t>(block_prefix[S]) * H) <=
                        checkpoint_capacity ? 1 : 0;
  }
  __syncthreads();
  int running = partial[threadIdx.x];
  for (int s = first; s < last; ++s) {
    block_prefix[s] = running;
    running += (seq_len[s] + 63) >> 6;
  }
}

// ---------------------------------------------------------------------------
// sign packing (wave64 ballot)
// ---------------------------------------------------------------------------

// Each lane reads one element of query and key; one 64-bit ballot then holds
// 64 / D complete symbols, which the first 64 / D lanes write out head-major.
template <int DTYPE>
__global__ __launch_bounds__(256) void pack_symbols_ballot_kernel(
    const void* __restrict__ query, const void* __restrict__ key,
    int32_t* __restrict__ packed_query, int32_t* __restrict__ packed_key, int64_t elements,
    int D, int H, int T, int N, int varlen) {
  const int64_t element = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool in_range = element < elements;
  const bool q_bit = in_range && load_as_float<DTYPE>(query, element) > 0.0f;
  const bool k_bit = in_range && load_as_float<DTYPE>(key, element) > 0.0f;
  const uint64_t q_mask = __ballot(q_bit);
  const uint64_t k_mask = __ballot(k_bit);
  const int lane = threadIdx.x & 63;
  const int symbols_per_wave = 64 / D;
  if (lane < symbols_per_wave) {
    const int64_t wave_first = element - lane;       // multiple of 64, hence of D
    const int64_t row = wave_first / D + lane;       // row = token * H + h
    if (row * D < elements) {
      const uint32_t field = D == 32 ? 0xffffffffu : ((1u << D) - 1u);
      const uint32_t q_word = static_cast<uint32_t>(q_mask >> (lane * D)) & field;
      const uint32_t k_word = static_cast<uint32_t>(k_mask >> (lane * D)) & field;
      const int64_t token = row / H;
      const int h = static_cast<int>(row - token * H);
      int64_t dst;
      if (varlen) {
        dst = static_cast<int64_t>(h) * N + token;
      } else {
        const int64_t b = token / T;
        dst = (b * H + h) * T + (token - b * T);
      }
      packed_query[dst] = static_cast<int32_t>(q_word);
      packed_key[dst] = static_cast<int32_t>(k_word);
    }
  }
}

// Widths that do not divide 64: one lane per symbol.
template <int DTYPE>
__global__ __launch_bounds__(256) void pack_symbols_rows_kernel(
    const void* __restrict__ query, const void* __restrict__ key,
    int32_t* __restrict__ packed_query, int32_t* __restrict__ packed_key, int64_t rows, int D,
    int H, int T, int N, int varlen) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  uint32_t q_word = 0u, k_word = 0u;
  for (int bit = 0; bit < D; ++bit) {
    if (load_as_float<DTYPE>(query, row * D + bit) > 0.0f) q_word |= 1u << bit;
    if (load_as_float<DTYPE>(key, row * D + bit) > 0.0f) k_word |= 1u << bit;
  }
  const int64_t token = row / H;
  const int h = static_cast<int>(row - token * H);
  int64_t dst;
  if (varlen) {
    dst = static_cast<int64_t>(h) * N + token;
  } else {
    const int64_t b = token / T;
    dst = (b * H + h) * T + (token - b * T);
  }
  packed_query[dst] = static_cast<int32_t>(q_word);
  packed_key[dst] = static_cast<int32_t>(k_word);
}

// ---------------------------------------------------------------------------
// hard forward: latest-longest route per row
// ---------------------------------------------------------------------------

// One wave owns 64 consecutive rows (lane = row) and walks over routes a.
// The run length obeys run(t, a) = eq(t, a) ? min(run(t-1, a-1) + 1, W) : 0;
// run(t-1, a-1) is the previous step's value of the lane above, fetched with
// one DPP shift.  Lane 0 has no lane above: its predecessor row t0-1 is
// evaluated directly, 64 routes at a time, by an early-exit compare loop.
// The winner is "longest first, latest on ties"; a zero run never produces a route.
// Both scans serve the training forward (32-bit symbol words) and the streaming router
// (byte symbols): `q` and `k` are the symbols of one (sequence, head), `length` rows long.
struct RouteWinner {
  int run;    // matched suffix length, 0 if no route matched
  int route;  // a, meaningful when run > 0
};

// run length of route `column` on row t0 - 1 (the row above the block), for lane 0
template <typename Symbol>
__device__ __forceinline__ int halo_run(const Symbol* q, const Symbol* k, int t0, int column,
                                        int W) {
  int halo = 0;
  if (column >= 1 && column <= t0 - 1) {
    const int limit = min(W, column);
    while (halo < limit && q[t0 - 1 - halo] == k[column - 1 - halo]) ++halo;
  }
  return halo;
}

// Any length: the winner is the maximum of the 64-bit key (run << 32) | a.
template <typename Symbol>
__device__ __forceinline__ RouteWinner scan_routes_wide(const Symbol* q, const Symbol* k, int t0,
                                                        int length, int W, int lane,
                                                        uint32_t q_symbol) {
  const int t = t0 + lane;
  const int a_last = min(t0 + kWave - 1, length - 1);
  uint64_t best = 0;
  int run = 0;
  for (int a0 = 1; a0 <= a_last; a0 += kWave) {
    const int column = a0 - 1 + lane;  // route index on the predecessor row t0 - 1
    const int halo = halo_run(q, k, t0, column, W);
    const uint32_t key_chunk = column < length ? k[column] : 0u;  // key symbol of route a0 + lane
    const int count = min(kWave, a_last - a0 + 1);
    for (int j = 0; j < count; ++j) {
      const uint32_t k_symbol = __builtin_amdgcn_readlane(key_chunk, j);
      const int halo_j = __builtin_amdgcn_readlane(halo, j);
      const int above = dpp_wave_shr1(halo_j, run);
      const int a = a0 + j;
      const bool match = (q_symbol == k_symbol) && (a <= t);
      run = match ? min(above + 1, W) : 0;
      best = max(best, (static_cast<uint64_t>(run) << 32) | static_cast<uint32_t>(a));
    }
  }
  return RouteWinner{static_cast<int>(best >> 32), static_cast<int>(best & 0xffffffffu)};
}

// length < 2^shift and W < 2^(32 - shift).  The same recurrence on
// `missing` = (W - run) << shift, so that the step is one saturating subtraction and the
// key needs no shift: the winner is the *minimum* of missing | (low - a).  Chunks of 64
// routes that lie entirely below the row block need no causal mask and are unrolled.
//
// On symbols of six or more random bits most steps match in no row of the wave (with 8 bits
// 78 % of them): such a step leaves every run at zero and cannot improve a winner, so an
// unmasked chunk runs in one of two forms.  The sparse form compares (one vector
// instruction against the key symbol in a scalar register) and skips the step when no lane
// matched; the update is done only on a step with a match, after the runs have been set to
// zero if the step before it was skipped.  The dense form is the plain update of every
// step.  Each chunk counts its steps with a match and the next chunk takes the form that
// suits that count, so match-dense inputs (few symbol bits, repeated motifs) keep the dense
// walk.
constexpr int kDenseChunkHits = 52;  // steps with a match (of 64) from which the dense form pays

template <typename Symbol>
__device__ __forceinline__ RouteWinner scan_routes_narrow(const Symbol* q, const Symbol* k,
                                                          int t0, int length, int W, int shift,
                                                          int lane, uint32_t q_symbol) {
  const int t = t0 + lane;
  const int a_last = min(t0 + kWave - 1, length - 1);
  const uint32_t one = 1u << shift;
  const uint32_t low = one - 1u;
  const uint32_t cap = static_cast<uint32_t>(W) << shift;
  uint32_t best = cap | low;  // run 0
  uint32_t missing = cap;
  // symbol of the row above the block (lane 0's predecessor row), wave-uniform
  const uint32_t q_above = t0 >= 1 ? static_cast<uint32_t>(q[t0 - 1]) : 0u;
  // key symbols of a chunk are fetched one chunk ahead: key position `column` (route
  // column + 1) and the position before it, which decides whether the halo run is non-zero
  uint32_t next_key = lane < length ? static_cast<uint32_t>(k[lane]) : 0u;
  uint32_t next_before = (lane >= 1 && lane - 1 < length) ? static_cast<uint32_t>(k[lane - 1]) : 0u;
  int hits = 0;  // steps with a match in the chunk before
  for (int a0 = 1; a0 <= a_last; a0 += kWave) {
    const int column = a0 - 1 + lane;
    const uint32_t key_chunk = next_key;
    const uint32_t key_before = next_before;
    {
      const int ahead = column + kWave;
      const bool wanted = a0 + kWave <= a_last;
      next_key = (wanted && ahead < length) ? static_cast<uint32_t>(k[ahead]) : 0u;
      next_before = (wanted && ahead - 1 < length) ? static_cast<uint32_t>(k[ahead - 1]) : 0u;
    }
    // run of route `column` on the row above the block: non-zero only where the first
    // symbols agree, which the registers decide; the rare longer compare reads memory
    int halo = 0;
    if (column >= 1 && column <= t0 - 1 && key_before == q_above) {
      const int limit = min(W, column);
      halo = 1;
      while (halo < limit && q[t0 - 1 - halo] == k[column - 1 - halo]) ++halo;
    }
    const uint32_t halo_missing = cap - (static_cast<uint32_t>(halo) << shift);
    const uint32_t route_low = low - static_cast<uint32_t>(a0);
    if (a0 + kWave - 1 <= t0) {
      if (hits < kDenseChunkHits) {
        hits = 0;
        int last_hit = -1;  // step that last updated the runs (they are valid when a chunk starts)
        const Symbol* key_symbols = k + (a0 - 1);
        constexpr int kBatch = 16;  // key symbols held in scalar registers at a time
        uint32_t batch[kBatch], batch_ahead[kBatch];
        const auto load_batch = [&](uint32_t (&into)[kBatch], int first) {
          // wave-uniform addresses: scalar loads
#pragma unroll
          for (int e = 0; e < kBatch; ++e) into[e] = key_symbols[first + e];
        };
        const auto arrive = [&](uint32_t (&held)[kBatch]) {
#pragma unroll
          for (int e = 0; e < kBatch; e += 8) {
            asm volatile("" : "+s"(held[e]), "+s"(held[e + 1]), "+s"(held[e + 2]), "+s"(held[e + 3]),
                              "+s"(held[e + 4]), "+s"(held[e + 5]), "+s"(held[e + 6]), "+s"(held[e + 7]));
          }
        };
        if constexpr (sizeof(Symbol) == 4) load_batch(batch, 0);
#pragma unroll
        for (int j0 = 0; j0 < kWave; j0 += kBatch) {
          if constexpr (sizeof(Symbol) == 4) {
            // the batch is taken in here, and only then does the next one set out: a wait for
            // scalar loads is a wait for all of them
            arrive(batch);
            if (j0 + kBatch < kWave) load_batch(batch_ahead, j0 + kBatch);
          }
#pragma unroll
          for (int e = 0; e < kBatch; ++e) {
            const int j = j0 + e;
            uint32_t k_symbol;
            if constexpr (sizeof(Symbol) == 4) {
              k_symbol = batch[e];
            } else {
              k_symbol = __builtin_amdgcn_readlane(key_chunk, j);
            }
            const bool match = q_symbol == k_symbol;
            if (__builtin_amdgcn_ballot_w64(match) != 0ull) {
              if (last_hit != j - 1) missing = cap;  // skipped steps left every run at zero
              const uint32_t above = dpp_wave_shr1(
                  static_cast<uint32_t>(__builtin_amdgcn_readlane(halo_missing, j)), missing);
              missing = match ? __builtin_elementwise_sub_sat(above, one) : cap;
              best = min(best, missing | (route_low - static_cast<uint32_t>(j)));
              last_hit = j;
              ++hits;
            }
          }
          if constexpr (sizeof(Symbol) == 4) {
#pragma unroll
            for (int e = 0; e < kBatch; ++e) batch[e] = batch_ahead[e];
          }
        }
        if (last_hit != kWave - 1) missing = cap;
      } else {
        // (the steps with a match are counted on every eighth step)
        hits = 0;
#pragma unroll
        for (int j = 0; j < kWave; ++j) {
          const uint32_t k_symbol = __builtin_amdgcn_readlane(key_chunk, j);
          const uint32_t above = dpp_wave_shr1(
              static_cast<uint32_t>(__builtin_amdgcn_readlane(halo_missing, j)), missing);
          const bool match = q_symbol == k_symbol;
          if (j % 8 == 0) hits += __builtin_amdgcn_ballot_w64(match) != 0ull ? 8 : 0;
          missing = match ? __builtin_elementwise_sub_sat(above, one) : cap;
          best = min(best, missing | (route_low - static_cast<uint32_t>(j)));
        }
      }
    } else {
      const int count = min(kWave, a_last - a0 + 1);
      for (int j = 0; j < count; ++j) {
        const uint32_t k_symbol = __builtin_amdgcn_readlane(key_chunk, j);
        const uint32_t above = dpp_wave_shr1(
            static_cast<uint32_t>(__builtin_amdgcn_readlane(halo_missing, j)), missing);
        const bool match = (q_symbol == k_symbol) && (a0 + j <= t);
        missing = match ? __builtin_elementwise_sub_sat(above, one) : cap;
        best = min(best, missing | (route_low - static_cast<uint32_t>(j)));
      }
    }
  }
  return RouteWinner{W - static_cast<int>(best >> shift), static_cast<int>(low - (best & low))};
}

template <bool VARLEN, bool WIDE>
__global__ __launch_bounds__(kWave) void hard_route_kernel(
    Layout L, const uint32_t* __restrict__ packed_query,
    const uint32_t* __restrict__ packed_key, int32_t* __restrict__ routes,
    int32_t* __restrict__ lengths, int32_t* __restrict__ source_token, int shift) {
  const Unit u = decode_unit<VARLEN>(L, blockIdx.x);
  if (!u.valid) return;
  const int blocks = (u.len + 63) >> 6;
  if (u.block >= blocks) return;
  const int row_block = blocks - 1 - u.block;  // longest rows are scheduled first
  const int t0 = row_block * kWave;
  const int lane = threadIdx.x;
  const uint32_t* q = packed_query + u.word_base;
  const uint32_t* k = packed_key + u.word_base;
  const int t = t0 + lane;
  const bool row_ok = t < u.len;
  const uint32_t q_word = row_ok ? q[t] : 0u;
  const RouteWinner winner = WIDE ? scan_routes_wide(q, k, t0, u.len, L.W, lane, q_word)
                                  : scan_routes_narrow(q, k, t0, u.len, L.W, shift, lane, q_word);
  if (!row_ok) return;
  const int route = winner.run > 0 ? winner.route : 0;
  if (routes != nullptr) routes[u.word_base + t] = route;
  if (lengths != nullptr) lengths[u.word_base + t] = winner.run;
  source_token[u.word_base + t] = route > 0 ? u.start + route : -1;
}

// output[token, h, :] = sign(value[source, h / group, :]) or exact zero.  `offset_error`
// (packed layout only, else NULL) points at the flag of invalid cu_seqlens: when it is set
// no row was routed and every output element becomes NaN, so that the mistake cannot pass
// for a result.
template <int DTYPE>
__global__ __launch_bounds__(256) void gather_values_kernel(
    const int32_t* __restrict__ source_token, const void* __restrict__ value,
    void* __restrict__ output, int64_t elements, int H, int Hv, int Dv, int T, int N,
    int varlen, const int32_t* __restrict__ offset_error) {
  const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= elements) return;
  if (offset_error != nullptr && *offset_error != 0) {
    store_nan<DTYPE>(output, index);
    return;
  }
  const int d = static_cast<int>(index % Dv);
  const int64_t row = index / Dv;
  const int h = static_cast<int>(row % H);
  const int64_t token = row / H;
  int64_t word;
  if (varlen) {
    word = static_cast<int64_t>(h) * N + token;
  } else {
    const int64_t b = token / T;
    word = (b * H + h) * T + (token - b * T);
  }
  const int source = source_token[word];
  int sign = 0;
  if (source >= 0) {
    const int hv = h / (H / Hv);
    const float x = load_as_float<DTYPE>(
        value, (static_cast<int64_t>(source) * Hv + hv) * Dv + d);
    sign = x > 0.0f ? 1 : -1;
  }
  store_sign<DTYPE>(output, index, sign);
}

// The same output as sign and validity bits, for a consumer that expands the ternary
// values itself (the prologue of the projection that follows the operator): per
// (token, head) ceil(Dv / 32) words whose bit d is value[source, hv, d] > 0, zero for the
// null route, and one byte that is 1 when a route was selected.  One thread per word.
template <int DTYPE>
__global__ __launch_bounds__(256) void gather_value_bits_kernel(
    const int32_t* __restrict__ source_token, const void* __restrict__ value,
    uint32_t* __restrict__ sign_words, uint8_t* __restrict__ routed, int64_t words, int H,
    int Hv, int Dv, int nvw, int T, int N, int varlen,
    const int32_t* __restrict__ offset_error) {
  const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= words) return;
  const int w = static_cast<int>(index % nvw);
  const int64_t row = index / nvw;  // token * H + h
  const int h = static_cast<int>(row % H);
  const int64_t token = row / H;
  if (offset_error != nullptr && *offset_error != 0) {
    // invalid cu_seqlens: bits cannot carry NaN; validity 0xff is the marker
    sign_words[index] = 0u;
    if (w == 0) routed[row] = uint8_t(0xff);
    return;
  }
  int64_t word_index;
  if (varlen) {
    word_index = static_cast<int64_t>(h) * N + token;
  } else {
    const int64_t b = token / T;
    word_index = (b * H + h) * T + (token - b * T);
  }
  const int source = source_token[word_index];
  uint32_t bits = 0u;
  if (source >= 0) {
    const int hv = h / (H / Hv);
    const int64_t base = (static_cast<int64_t>(source) * Hv + hv) * Dv + 32 * w;
    const int count = min(32, Dv - 32 * w);
    for (int d = 0; d < count; ++d) {
      if (load_as_float<DTYPE>(value, base + d) > 0.0f) bits |= 1u << d;
    }
  }
  sign_words[index] = bits;
  if (w == 0) routed[row] = source >= 0 ? uint8_t(1) : uint8_t(0);
}

// Sign symbols of a contiguous [rows][bits] tensor in the order of its rows: bit i of the
// symbol is x[row, i] > 0.  OUT is uint8_t (bits <= 8, the streaming router's symbols) or
// uint32_t.  Widths that divide 64 take one lane per element and one ballot per 64
// elements; other widths take one lane per row.
template <int DTYPE, typename OUT>
__global__ __launch_bounds__(256) void pack_rows_ballot_kernel(const void* __restrict__ logits,
                                                               OUT* __restrict__ symbols,
                                                               int64_t elements, int bits) {
  const int64_t element = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool positive = element < elements && load_as_float<DTYPE>(logits, element) > 0.0f;
  const uint64_t mask = __ballot(positive);
  const int lane = threadIdx.x & 63;
  if (lane < 64 / bits) {
    const int64_t row = (element - lane) / bits + lane;
    if (row * bits < elements) {
      const uint32_t field = bits == 32 ? 0xffffffffu : ((1u << bits) - 1u);
      symbols[row] = static_cast<OUT>(static_cast<uint32_t>(mask >> (lane * bits)) & field);
    }
  }
}

template <int DTYPE, typename OUT>
__global__ __launch_bounds__(256) void pack_rows_serial_kernel(const void* __restrict__ logits,
                                                               OUT* __restrict__ symbols,
                                                               int64_t rows, int bits) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  uint32_t symbol = 0u;
  for (int bit = 0; bit < bits; ++bit) {
    if (load_as_float<DTYPE>(logits, row * bits + bit) > 0.0f) symbol |= 1u << bit;
  }
  symbols[row] = static_cast<OUT>(symbol);
}

// ---------------------------------------------------------------------------
// backward: preparation
// ---------------------------------------------------------------------------

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

// grad_output -> head-major rows of bfloat16 terms, [row][term][dvp] padded with zeros to
// whole blocks of 32 elements (`pitch` elements per row).  One thread per (row, value
// dimension of the padded width): loads are runs of Dv elements, stores of one term are
// contiguous over the threads of a row.
template <int DTYPE>
__device__ __forceinline__ void prepare_grad_rows(
    int64_t index, const void* __restrict__ grad_output, uint16_t* __restrict__ grad_rows,
    int64_t rows, int H, int Dv, int dvp, int T, int N, int varlen, int value_stride,
    int value_offset, int terms, int pitch) {
  if (index >= rows * dvp) return;
  const int64_t dst = index / dvp;  // head-major row
  const int d = static_cast<int>(index - dst * dvp);
  int64_t source_row;  // token * H + h
  if (varlen) {
    const int64_t h = dst / N;
    source_row = (dst - h * N) * H + h;
  } else {
    const int64_t bh = dst / T;
    const int64_t b = bh / H;
    source_row = (b * T + (dst - bh * T)) * H + (bh - b * H);
  }
  float rest =
      d < Dv ? load_as_float<DTYPE>(grad_output, source_row * value_stride + value_offset + d)
             : 0.0f;
  uint16_t* row = grad_rows + dst * pitch;
  for (int t = 0; t < terms; ++t) {
    const uint32_t term = bf16_nearest(rest);
    row[t * dvp + d] = static_cast<uint16_t>(term);
    // exact: the term holds the leading bits of `rest`; an infinite or NaN term ends the series
    rest = (term & 0x7f80u) == 0x7f80u ? 0.0f : rest - __uint_as_float(term << 16);
  }
  for (int k = terms * dvp + d; k < pitch; k += dvp) row[k] = uint16_t(0);
}

__device__ __forceinline__ int64_t value_word_row(int64_t row, int Hv, int T, int N, int varlen) {
  const int64_t token = row / Hv;  // row = token * Hv + hv
  const int64_t hv = row - token * Hv;
  if (varlen) return hv * N + token;
  const int64_t b = token / T;
  return (b * Hv + hv) * T + (token - b * T);
}

// Value sign bits for widths 8, 16, 32 and 64: one lane per element in the order of the
// tensor, one wave ballot per 64 elements; the lane at the start of a 32-bit group (or of
// a narrower row) stores that group's word.  Every lane of the wave must call this.
template <int DTYPE>
__device__ __forceinline__ void pack_value_bits_ballot(
    int64_t index, const void* __restrict__ value, uint32_t* __restrict__ value_bits,
    int64_t rows, int Hv, int Dv, int nvw, int T, int N, int varlen, int value_stride,
    int value_offset) {
  const bool inside = index < rows * Dv;
  const int64_t row = index / Dv;
  const int d = static_cast<int>(index - row * Dv);
  const bool positive =
      inside && load_as_float<DTYPE>(value, row * value_stride + value_offset + d) > 0.0f;
  const uint64_t ballot = __ballot(positive);
  if (inside && (d & 31) == 0) {
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t word = static_cast<uint32_t>(ballot >> lane);
    if (Dv < 32) word &= (1u << Dv) - 1u;
    value_bits[value_word_row(row, Hv, T, N, varlen) * nvw + (d >> 5)] = word;
  }
}

// value sign bits, head-major over value heads: word index (seq, hv, t) like the symbol words
// (any width: one thread per row)
template <int DTYPE>
__device__ __forceinline__ void pack_value_bits_rows(
    int64_t row, const void* __restrict__ value, uint32_t* __restrict__ value_bits, int64_t rows,
    int Hv, int Dv, int nvw, int T, int N, int varlen, int value_stride, int value_offset) {
  if (row >= rows) return;  // row = token * Hv + hv
  const int64_t dst = value_word_row(row, Hv, T, N, varlen);
  for (int w = 0; w < nvw; ++w) {
    uint32_t word = 0u;
    for (int bit = 0; bit < 32; ++bit) {
      const int d = w * 32 + bit;
      if (d < Dv && load_as_float<DTYPE>(value, row * value_stride + value_offset + d) > 0.0f) {
        word |= 1u << bit;
      }
    }
    value_bits[dst * nvw + w] = word;
  }
}

// Per row: the reference point of the softmax exponent and the constant part
// of the logit.  With `analytic` the reference point is the upper bound
// max(null, scale*U(min(W, t)) - log t) of every logit of the row, otherwise it
// starts at the null logit and a separate pass raises it to the row maximum.
template <bool VARLEN>
__device__ __forceinline__ void init_row_stats(int64_t index, const Layout& L,
                                               float4* __restrict__ stats, float scale,
                                               int analytic, int32_t* __restrict__ work_counter) {
  if (index == 0) {
    work_counter[0] = 0;
    work_counter[3] = 0;  // header word 4: a long match was met
  }
  const int64_t rows = static_cast<int64_t>(L.N) * L.H;
  if (index >= rows) return;
  // head-major index -> local row t
  int t;
  if constexpr (VARLEN) {
    const int token = static_cast<int>(index % L.N);
    int low = 0, high = L.S;  // sequence containing the token (empty sequences are skipped)
    while (low < high) {
      const int mid = (low + high) >> 1;
      if (L.seq_start[mid] + L.seq_len[mid] <= token) low = mid + 1; else high = mid;
    }
    t = low < L.S ? token - L.seq_start[low] : 0;
    if (t < 0) t = 0;
  } else {
    t = static_cast<int>(index % L.T);
  }
  const float null_logit = kNullScore * scale;
  const float log_count = t > 0 ? logf(static_cast<float>(t)) : 0.0f;
  float reference = null_logit;
  if (analytic) {
    const float longest = static_cast<float>(min(L.W, t));
    const float bound = scale * kSqrtScale * (sqrtf(1.0f + longest) - 1.0f) - log_count;
    reference = fmaxf(null_logit, bound);
  }
  const float base = (scale * kSqrtScale + log_count) * kLog2e;
  stats[index] = make_float4(reference, 0.0f, 0.0f, base);
}

// Everything the two backward passes need before they start, as one launch: the four
// parts are independent and own consecutive ranges of the grid.
struct PrepareParams {
  Layout L;
  const void* grad_output;
  const void* value;
  uint16_t* grad_rows;
  uint32_t* value_bits;
  float4* stats;
  int32_t* work_counter;
  int64_t symbol_rows, value_rows;
  int Dv, dvp, nvw, value_stride, value_offset;
  int grad_terms, grad_pitch;  // bfloat16 terms per grad_output element, elements per row
  float scale;
  int analytic;
  int ballot;  // value width is 8, 16, 32 or 64: pack signs with wave ballots
  float* fill[3];  // gradient buffers to clear (null: none), with their lengths
  int64_t fill_elements[3];
  unsigned grad_blocks, value_blocks, stats_blocks, fill_blocks;
};

template <int DTYPE, bool VARLEN>
__global__ __launch_bounds__(256) void vjp_prepare_kernel(PrepareParams p) {
  unsigned block = blockIdx.x;
  const auto element = [&]() { return static_cast<int64_t>(block) * blockDim.x + threadIdx.x; };
  if (block < p.grad_blocks) {
    prepare_grad_rows<DTYPE>(element(), p.grad_output, p.grad_rows, p.symbol_rows, p.L.H, p.Dv,
                             p.dvp, p.L.T, p.L.N, p.L.varlen, p.value_stride, p.value_offset,
                             p.grad_terms, p.grad_pitch);
    return;
  }
  block -= p.grad_blocks;
  if (block < p.value_blocks) {
    if (p.ballot) {
      pack_value_bits_ballot<DTYPE>(element(), p.value, p.value_bits, p.value_rows, p.L.Hv, p.Dv,
                                    p.nvw, p.L.T, p.L.N, p.L.varlen, p.value_stride,
                                    p.value_offset);
    } else {
      pack_value_bits_rows<DTYPE>(element(), p.value, p.value_bits, p.value_rows, p.L.Hv, p.Dv,
                                  p.nvw, p.L.T, p.L.N, p.L.varlen, p.value_stride,
                                  p.value_offset);
    }
    return;
  }
  block -= p.value_blocks;
  if (block < p.stats_blocks) {
    init_row_stats<VARLEN>(element(), p.L, p.stats, p.scale, p.analytic, p.work_counter);
    return;
  }
  block -= p.stats_blocks;
  const int64_t stride = static_cast<int64_t>(p.fill_blocks) * blockDim.x;
  for (int part = 0; part < 3; ++part) {
    if (p.fill[part] == nullptr) continue;
    for (int64_t i = element(); i < p.fill_elements[part]; i += stride) p.fill[part][i] = 0.0f;
  }
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

// After the row-statistics pass a row's float4 (reference, denominator, dropped
// utility sum, constant logit part) is replaced by what the gradient pass reads per
// row: (unused, exponent shift including log2 of the denominator, expected dropped
// utility, unused).
__global__ __launch_bounds__(256) void finalize_row_records_kernel(float4* __restrict__ stats,
                                                                   int64_t rows,
                                                                   float null_logit) {
  const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= rows) return;
  const float4 row = stats[index];
  const float denominator = row.y + fast_exp2((null_logit - row.x) * kLog2e);
  uint4 record;
  record.x = 0u;
  record.y = __float_as_uint(fmaf(row.x, kLog2e, row.w) + __log2f(denominator));
  record.z = __float_as_uint(row.z / denominator);
  record.w = 0u;
  reinterpret_cast<uint4*>(stats)[index] = record;
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
constexpr int gradient_waves(int value_tiles, int symbol_tiles) {
  if (value_tiles == 1 && symbol_tiles == 1) return 3;
  if (value_tiles == 4 && symbol_tiles == 2) return 1;   // 120 accumulator registers alone
  return 2;
}

// rows staged in LDS per segment of the gradient kernel (a multiple of kChunk): with 32 a
// single-wave block of the narrowest tile needs 11.4 KB, which leaves room for three per SIMD
constexpr int gradient_segment(int /*dvp*/) { return 32; }

// resident waves of the persistent gradient kernel per wave it is compiled to hold on each
// SIMD of the 256 compute units
constexpr int kMaxResidentBlocks = 2048;  // at two waves per SIMD
constexpr int resident_gradient_waves(int value_tiles, int symbol_tiles) {
  return 1024 * (gradient_waves(value_tiles, symbol_tiles) < 2
                     ? 2 : gradient_waves(value_tiles, symbol_tiles));
}

// Waves per block of the gradient kernel (rosa_hip_set_gradient_block_waves overrides).
// Two waves halve the column atomics, which bound the wide tiles; the narrow tile is bound
// by its arithmetic, and with few bands per resident wave the kernel's time is that of
// its longest band, which a block of two waves walks more slowly than a single wave.
int g_gradient_block_waves = 0;  // 0: by shape


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

// How the gradient kernel is launched for a tile shape: waves per block, whether row tiles
// are queued between the bands of a block, and the LDS of a block.
struct GradientBlockPlan {
  int waves;
  bool row_queue;
  size_t wave_floats, tile_floats, lds_bytes;
};

int gradient_block_waves(int dvp, int symbol_tiles, int64_t units) {
  if (g_gradient_block_waves == 1 || g_gradient_block_waves == 2) return g_gradient_block_waves;
  return ((dvp >= 16 || symbol_tiles > 1) && units >= 2 * kMaxResidentBlocks) ? 2 : 1;
}

GradientBlockPlan plan_gradient_blocks(int dvp, int D, int value_words_per_column, int grad_pitch,
                                       int64_t units) {
  const int segment = gradient_segment(dvp);
  const int value_tiles = (dvp + 15) / 16;
  const int symbol_tiles = D > 16 ? 2 : 1;
  GradientBlockPlan plan;
  plan.wave_floats = gradient_wave_floats(dvp, grad_pitch);
  plan.tile_floats = exchange_tile_floats(dvp == 8 && D <= 8);
  // two waves: column tiles on their way to the other wave and, where the block stays within
  // its budget, the queue of row tiles
  if (gradient_block_waves(dvp, symbol_tiles, units) == 2) {
    size_t shared = gradient_shared_fixed_floats(segment, value_words_per_column, 2) +
                    (value_tiles + symbol_tiles) * plan.tile_floats;
    const size_t queue = kQueueSlots * symbol_tiles * plan.tile_floats;
    plan.row_queue =
        (2 * plan.wave_floats + shared + queue) * sizeof(float) <= kGradientBlockLdsBudget;
    if (plan.row_queue) shared += queue;
    plan.lds_bytes = (2 * plan.wave_floats + shared) * sizeof(float);
    if (plan.lds_bytes <= 64 * 1024) {
      plan.waves = 2;
      return plan;
    }
  }
  plan.waves = 1;  // also where two waves would not fit (float32 rows of the widest tile)
  plan.row_queue = false;
  plan.lds_bytes =
      (plan.wave_floats + gradient_shared_fixed_floats(segment, value_words_per_column, 1)) *
      sizeof(float);
  return plan;
}

// TERMS: bfloat16 terms that carry a gate adjoint into the symbol contractions.  Two terms
// hold it to 2^-18 of its size, which is enough where the terms of a gradient sum are of the
// size of the sum.  Long matches make them much larger than the sum (a row's adjoints
// cancel), so a launch in which the row-statistics pass has met a long match (evidence of
// kLongMatchEvidence at the end of a chunk, or an overflow term that matters: header word 4)
// runs the three-term form, 2^-21 by truncation; both forms are launched and the one that
// does not apply returns at once.
template <int NVW, int DVP, int DT, bool VARLEN, bool DROPOUT, int NW, int TERMS>
__global__ __launch_bounds__(kWave * NW)
__attribute__((amdgpu_waves_per_eu(gradient_waves((DVP + 15) / 16, DT))))
void vjp_gradients_kernel(VjpParams P) {
  static_assert(NW == 1 || NW == 2, "blocks of one or two waves");
  static_assert(TERMS == 2 || TERMS == 3, "two or three terms per gate adjoint");
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
  float* ck_evidence = ring + static_cast<int64_t>(P.ring_rows) * kWave;   // [SEG_CHUNKS][64]
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
    const Unit lead = decode_unit<VARLEN>(P.L, unit_index);
    if (!lead.valid) continue;
    if (NW > 1 && lead.block % NW != 0) continue;
    const int lead_steps = lead.len - 1 - lead.block * kWave;
    if (lead_steps <= 0) continue;
    Unit u = lead;
    u.block += wave;
    BandView view;
    int hv;
    const bool have_band = make_view<NVW, VARLEN>(P, u, view, hv);
    const int my_steps = have_band ? view.steps : 0;  // a wave without a band only keeps step
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
    float gate_below = 0.0f;      // gate of the row below
    float ring_sum = 0.0f;        // sum of b * overflow over the next W + 1 rows
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
        if (want_q && (NW == 1 || done_flush_rows)) {
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

    for (int segment = lead_segments - 1; segment >= 0; --segment) {
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
        const bool cached = DROPOUT && stored;
        if (steady && chunk_quiet) {
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
        if (want_v) {
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
          const bool quiet = steady && chunk_quiet && ring_live == 0;
          if (quiet) {
            // no overflow term of the chunk can move a gradient and the ring is empty:
            // h = b (S + o), nothing to mask
#pragma unroll
            for (int r = kChunk - 1; r >= 0; --r) {
              const float b = fmaf(gate_below, adjoint_carry, keep_adjoint[r]);
              adjoint_carry = b;
              gate_below = keep_gate[r];
              if constexpr (TERMS == 2) {
                tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16(b * keep_evidence[r]);
              } else {
                uint32_t rest;
                tile_bits[r * (kTilePitch + 1) + 64 - lane] = split_bf16_exact(b * keep_evidence[r], rest);
                rest_plane[r * (kRestPitch + 1) + 64 - lane] = static_cast<uint16_t>(rest >> 16);
              }
            }
          } else {
#pragma unroll
          for (int r = kChunk - 1; r >= 0; --r) {
            const int i = first + r;
            const float b = fmaf(gate_below, adjoint_carry, keep_adjoint[r]);
            adjoint_carry = b;
            gate_below = keep_gate[r];
            const float overflow = keep_overflow[r];
            const float term = overflow >= P.tail_threshold ? b * overflow : 0.0f;
            const bool any_term = __ballot(term != 0.0f) != 0ull;
            if (any_term) {
              if (ring_live == 0) ring_fresh = P.ring_rows;
              ring_live = P.ring_rows;
            }
            if (ring_live > 0) {
              const int slot = i % P.ring_rows;
              float leaving = 0.0f;
              if (ring_fresh > 0) {
                --ring_fresh;
              } else {
                leaving = ring[slot * kWave + lane];
              }
              ring[slot * kWave + lane] = term;
              ring_sum += term - leaving;
              --ring_live;
            }
            const float h = fmaf(b, keep_evidence[r], -ring_sum);
            if (ring_live == 0) ring_sum = 0.0f;
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

          if (want_k) {
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
          if (want_q) {
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
  }
}

// Softsign Jacobian 1 / (1 + |x|)^2 applied once to the symbol-space sums.
// Where the sums of a gradient tensor come from when they were accumulated head-major.
struct HeadMajorSums {
  const float* query;  // [sequence, head][position][D], row t stored at t - 1; NULL: in place
  const float* key;    // [sequence, head][position][D]
  const float* value;  // [sequence, value head][position][Dv], row a stored at a - 1
  int H, Hv, D, Dv, T, N, varlen;
};

// head-major row of (token, head) in a tensor with `heads` heads
__device__ __forceinline__ int64_t head_major_row(int64_t token, int head, int heads, int T,
                                                  int N, int varlen) {
  if (varlen) return static_cast<int64_t>(head) * N + token;
  const int64_t batch = token / T;
  return (batch * heads + head) * T + (token - batch * T);
}

template <int DTYPE>
__global__ __launch_bounds__(256) void finalize_gradients_kernel(
    const void* __restrict__ query, const void* __restrict__ key,
    const void* __restrict__ value, float* __restrict__ grad_query,
    float* __restrict__ grad_key, float* __restrict__ grad_value, int64_t symbol_elements,
    int64_t value_elements, const int32_t* __restrict__ offset_error, HeadMajorSums sums) {
  const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (offset_error != nullptr && *offset_error != 0) {
    // invalid cu_seqlens (packed layout): nothing was accumulated; every gradient is NaN
    const float nan = __uint_as_float(0x7fc00000u);
    if (index < symbol_elements) {
      if (grad_query != nullptr) grad_query[index] = nan;
      if (grad_key != nullptr) grad_key[index] = nan;
    }
    if (index < value_elements && grad_value != nullptr) grad_value[index] = nan;
    return;
  }
  if (index < symbol_elements) {
    int64_t row = 0;
    int d = 0;
    if (sums.query != nullptr || sums.key != nullptr) {
      const int64_t token_head = index / sums.D;
      d = static_cast<int>(index - token_head * sums.D);
      const int64_t token = token_head / sums.H;
      row = head_major_row(token, static_cast<int>(token_head - token * sums.H), sums.H, sums.T,
                           sums.N, sums.varlen);
    }
    if (grad_query != nullptr) {
      const float den = 1.0f + fabsf(load_as_float<DTYPE>(query, index));
      // the slot below the first row of a run is the unused last slot of the run before it
      const float sum = sums.query == nullptr ? grad_query[index]
                        : (row > 0 ? sums.query[(row - 1) * sums.D + d] : 0.0f);
      grad_query[index] = sum * (1.0f / (den * den));
    }
    if (grad_key != nullptr) {
      const float den = 1.0f + fabsf(load_as_float<DTYPE>(key, index));
      const float sum = sums.key == nullptr ? grad_key[index] : sums.key[row * sums.D + d];
      grad_key[index] = sum * (1.0f / (den * den));
    }
  }
  if (index < value_elements && grad_value != nullptr) {
    const float den = 1.0f + fabsf(load_as_float<DTYPE>(value, index));
    float sum;
    if (sums.value == nullptr) {
      sum = grad_value[index];
    } else {
      const int64_t token_head = index / sums.Dv;
      const int d = static_cast<int>(index - token_head * sums.Dv);
      const int64_t token = token_head / sums.Hv;
      const int64_t row = head_major_row(token, static_cast<int>(token_head - token * sums.Hv),
                                         sums.Hv, sums.T, sums.N, sums.varlen);
      sum = row > 0 ? sums.value[(row - 1) * sums.Dv + d] : 0.0f;
    }
    grad_value[index] = sum * (1.0f / (den * den));
  }
}

// Measurement aid: the rate of global float atomics in the access pattern of the gradient
// flush.  Every wave adds 16 x 16 tiles (lane (li, lg) adds rows 4 lg .. 4 lg + 3 of column
// li, four instructions per tile) at pseudo-random rows of a buffer whose rows are
// `row_stride` floats apart; `columns` <= 16 lanes of every row are active.  One
// instruction touches four rows, i.e. four 64-byte segments.
__global__ __launch_bounds__(kWave) void atomic_rate_kernel(float* buffer, uint32_t rows,
                                                            uint32_t row_stride, int columns,
                                                            int tiles) {
  const int lane = threadIdx.x;
  const int li = lane & 15;
  const int lg = lane >> 4;
  uint32_t state = blockIdx.x * 2654435761u + 12345u;
  for (int tile = 0; tile < tiles; ++tile) {
    state = state * 1664525u + 1013904223u;
    const uint32_t first_row = (state >> 8) % (rows - 16u);
    if (li < columns) {
      float* base = buffer + static_cast<size_t>(first_row + 4 * lg) * row_stride + li;
#pragma unroll
      for (int e = 0; e < 4; ++e) atomicAdd(base + e * row_stride, 1.0f);
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

size_t align_up(size_t bytes) { return (bytes + 255) & ~static_cast<size_t>(255); }

struct ProblemView {
  Layout L;
  int64_t tokens;        // B*T or N
  int64_t symbol_rows;   // tokens * H
  int64_t value_rows;    // tokens * Hv
  int grad_terms;        // bfloat16 terms that represent a grad_output element exactly
};

int check_problem(const rosa_problem* p, ProblemView* out) {
  if (p == nullptr) return fail(1, "problem is NULL");
  if (p->dtype < ROSA_DTYPE_F32 || p->dtype > ROSA_DTYPE_BF16) return fail(1, "unsupported dtype");
  if (p->H < 1 || p->Hv < 1 || p->H % p->Hv != 0)
    return fail(1, "query heads must be a positive multiple of value heads");
  if (p->D < 1 || p->D > 32) return fail(1, "query/key bit dimension must be in [1, 32]");
  if (p->Dv < 1) return fail(1, "value dimension must be positive");
  if (p->W < 1) return fail(1, "max_suffix_length must be >= 1");
  Layout L;
  memset(&L, 0, sizeof(L));
  L.H = p->H; L.D = p->D; L.Hv = p->Hv; L.Dv = p->Dv; L.W = p->W;
  int64_t tokens;
  if (p->cu_seqlens != nullptr || p->S > 0) {
    if (p->cu_seqlens == nullptr || p->S < 1 || p->N < 1)
      return fail(1, "packed layout needs cu_seqlens, S >= 1 and N >= 1");
    L.varlen = 1; L.N = p->N; L.S = p->S; L.B = 0; L.T = 0;
    tokens = p->N;
    const int64_t slots = static_cast<int64_t>(p->N) / 64 + p->S;
    if (slots > INT32_MAX) return fail(1, "number of packed sequences is too large");
    L.slots = static_cast<int>(slots);
  } else {
    if (p->B < 1 || p->T < 1) return fail(1, "dense layout needs B >= 1 and T >= 1");
    tokens = static_cast<int64_t>(p->B) * p->T;
    if (tokens > INT32_MAX) return fail(1, "B * T must fit in int32");
    L.varlen = 0; L.B = p->B; L.T = p->T; L.N = static_cast<int>(tokens); L.S = 0;
    L.slots = p->B * ((p->T + 63) / 64);
  }
  if (tokens * p->H > INT32_MAX) return fail(1, "tokens * H must fit in int32");
  if (static_cast<int64_t>(L.slots) * p->H > INT32_MAX) return fail(1, "too many work units");
  const int bound = L.varlen ? L.N : L.T;
  if (L.W > bound) L.W = bound;
  out->L = L;
  out->grad_terms = p->dtype == ROSA_DTYPE_F32 ? 3 : (p->dtype == ROSA_DTYPE_F16 ? 2 : 1);
  out->tokens = tokens;
  out->symbol_rows = tokens * p->H;
  out->value_rows = tokens * p->Hv;
  return 0;
}

// Workspace carving shared by the size queries and the launches.
struct ForwardWorkspace {
  size_t header, seq_start, seq_len, block_prefix, source_token, total;
};

ForwardWorkspace carve_forward(const ProblemView& v) {
  ForwardWorkspace w;
  size_t cursor = 0;
  w.header = cursor; cursor += align_up(256);
  const size_t s = static_cast<size_t>(v.L.varlen ? v.L.S : 0);
  w.seq_start = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.seq_len = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.block_prefix = cursor; cursor += align_up(sizeof(int32_t) * (s + 1));
  w.source_token = cursor; cursor += align_up(sizeof(int32_t) * static_cast<size_t>(v.symbol_rows));
  w.total = cursor;
  return w;
}

constexpr int kValueSlice = 64;  // value dimensions one backward pass covers
constexpr int kNarrowRow = 8;    // gradient rows up to this many floats are accumulated head-major

// bytes of chunk records the backward workspace may hold unless the caller sets a limit:
// at most 4 GiB, and in a packed layout, whose sequence lengths the host does not know, at
// most 1.5 KiB per token and head (what sequences of about 6 000 tokens need with dropout;
// longer ones make the device fall back to rebuilding the evidence in the gradient pass)
constexpr size_t kDefaultRecordBudget = size_t(1) << 32;
constexpr size_t kPackedRecordBytesPerRow = 1536;
constexpr size_t kNoRecordBudget = static_cast<size_t>(-1);
size_t g_record_budget_bytes = kNoRecordBudget;  // set by rosa_hip_set_record_budget

int value_words(int Dv) { return (Dv + 31) / 32; }

int padded_value_width(int Dv) {
  if (Dv <= 8) return 8;
  if (Dv <= 16) return 16;
  if (Dv <= 32) return 32;
  return 64;
}

struct VjpWorkspace {
  size_t header, seq_start, seq_len, block_prefix, step_prefix, stats, grad_rows,
      value_bits, block_scratch, total;
  size_t sums_query, sums_key, sums_value;  // head-major accumulators (rows of <= 8 floats)
  bool symbols_by_head, values_by_head;
  size_t checkpoints;
  int64_t checkpoint_capacity;  // chunk records that fit in the workspace (0: none kept)
  int record_floats;
  int resident_blocks;
  int64_t block_scratch_floats;
  int segment_group;
  int ring_rows;
};


VjpWorkspace carve_vjp(const ProblemView& v, bool dropout) {
  VjpWorkspace w;
  size_t cursor = 0;
  w.header = cursor; cursor += align_up(256);
  const size_t s = static_cast<size_t>(v.L.varlen ? v.L.S : 0);
  w.seq_start = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.seq_len = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.block_prefix = cursor; cursor += align_up(sizeof(int32_t) * (s + 1));
  w.step_prefix = cursor; cursor += align_up(sizeof(int64_t) * (s + 1));
  const size_t rows = static_cast<size_t>(v.symbol_rows);
  const int slice_width = std::min(v.L.Dv, kValueSlice);
  const int dvp = padded_value_width(slice_width);
  w.stats = cursor; cursor += align_up(sizeof(float) * 4 * rows);
  w.grad_rows = cursor;
  cursor += align_up(sizeof(uint16_t) * rows * grad_term_pitch(v.grad_terms, dvp));
  w.value_bits = cursor;
  cursor += align_up(sizeof(uint32_t) * static_cast<size_t>(v.value_rows) * value_words(slice_width));
  // head-major accumulators for gradient rows of at most 8 floats (VjpParams::symbols_by_head)
  w.symbols_by_head = v.L.D <= kNarrowRow;
  w.values_by_head = v.L.Dv <= kNarrowRow;
  const size_t symbol_sums = w.symbols_by_head ? sizeof(float) * rows * v.L.D : 0;
  w.sums_query = cursor; cursor += align_up(symbol_sums);
  w.sums_key = cursor; cursor += align_up(symbol_sums);
  w.sums_value = cursor;
  cursor += align_up(w.values_by_head ? sizeof(float) * static_cast<size_t>(v.value_rows) * v.L.Dv : 0);
  // Chunk records written by the row-statistics pass for the gradient pass, which
  // otherwise rebuilds the evidence with forward sweeps of its own and evaluates the
  // dropout hash a second time.
  w.checkpoints = cursor;
  w.record_floats = kCheckpointFloats + (dropout ? kKeepBitFloats : 0);
  {
    size_t budget_bytes = g_record_budget_bytes;
    if (budget_bytes == kNoRecordBudget) {
      budget_bytes = kDefaultRecordBudget;
      if (v.L.varlen) budget_bytes = std::min(budget_bytes, kPackedRecordBytesPerRow * rows);
    }
    const int64_t budget = static_cast<int64_t>(budget_bytes / (sizeof(float) * w.record_floats));
    const int64_t steps = v.L.varlen
        ? static_cast<int64_t>(v.L.H) * band_steps_total(v.L.N)
        : static_cast<int64_t>(v.L.B) * v.L.H * band_steps_total(v.L.T);
    const int64_t wanted = checkpoint_slots(steps, static_cast<int64_t>(v.L.slots) * v.L.H);
    w.checkpoint_capacity = v.L.varlen ? std::min(wanted, budget) : (wanted <= budget ? wanted : 0);
    cursor += align_up(sizeof(float) * w.record_floats *
                       static_cast<size_t>(w.checkpoint_capacity));
  }
  const int longest = v.L.varlen ? v.L.N : v.L.T;
  w.ring_rows = std::min(v.L.W, longest) + 1;
  const int segment_rows = gradient_segment(dvp);
  // one fallback checkpoint per segment of the longest possible band, for a wave that finds
  // no records: never the case in a dense layout whose records fit (known here), decided on
  // the device in a packed one
  // (nor in one whose window counts the records can always hold: see the launch)
  const bool may_run_without_records =
      v.L.varlen != 0 || w.checkpoint_capacity == 0 ||
      (static_cast<int64_t>(w.ring_rows) * v.L.D > kRecordWindowMax);
  const int max_segments =
      may_run_without_records ? (longest + segment_rows - 1) / segment_rows + 1 : 0;
  // two levels: a checkpoint per group of G segments and one per segment of a group, with G
  // near the square root of the segment count
  w.segment_group = 4;
  while (w.segment_group * w.segment_group < max_segments) ++w.segment_group;
  const int max_groups = max_segments > 0 ? (max_segments + w.segment_group - 1) / w.segment_group : 0;
  w.block_scratch_floats = static_cast<int64_t>(w.ring_rows) * kWave +
                           2 * kCheckpointChunksMax * kWave +
                           static_cast<int64_t>(max_segments > 0 ? max_groups + w.segment_group : 0) *
                               2 * kWave;
  const int64_t units = static_cast<int64_t>(v.L.slots) * v.L.H;
  // resident waves of the gradient kernel (an even number: its blocks hold one or two waves)
  w.resident_blocks = static_cast<int>(std::min<int64_t>(
      (units + 1) & ~int64_t(1), resident_gradient_waves((dvp + 15) / 16, v.L.D > 16 ? 2 : 1)));
  // keep the scratch pool below 2 GiB by running fewer resident blocks for huge windows
  const int64_t budget_floats = (int64_t(1) << 31) / 4;
  while (w.resident_blocks > 64 &&
         static_cast<int64_t>(w.resident_blocks) * w.block_scratch_floats > budget_floats) {
    w.resident_blocks /= 2;
  }
  w.block_scratch = cursor;
  cursor += align_up(sizeof(float) * static_cast<size_t>(w.resident_blocks) *
                     static_cast<size_t>(w.block_scratch_floats));
  w.total = cursor;
  return w;
}

template <typename T>
T* at(void* base, size_t offset) {
  return reinterpret_cast<T*>(static_cast<char*>(base) + offset);
}

unsigned blocks_for(int64_t items, int threads) {
  return static_cast<unsigned>((items + threads - 1) / threads);
}

int launch_prepare_sequences(const rosa_problem* p, Layout& L, void* workspace, size_t seq_start,
                             size_t seq_len, size_t block_prefix, size_t header,
                             hipStream_t stream, int64_t* step_prefix = nullptr,
                             int64_t checkpoint_capacity = 0) {
  if (!L.varlen) return 0;
  L.seq_start = at<int32_t>(workspace, seq_start);
  L.seq_len = at<int32_t>(workspace, seq_len);
  L.block_prefix = at<int32_t>(workspace, block_prefix);
  L.step_prefix = step_prefix;
  hipLaunchKernelGGL(prepare_sequences_kernel, dim3(1), dim3(256), 0, stream, p->cu_seqlens, L.S,
                     L.N, at<int32_t>(workspace, seq_start), at<int32_t>(workspace, seq_len),
                     at<int32_t>(workspace, block_prefix), step_prefix, L.H, checkpoint_capacity,
                     at<int32_t>(workspace, header));
  return 0;
}

template <int DTYPE>
int run_forward(const rosa_problem* p, const ProblemView& view, const void* query,
                const void* key, const void* value, void* output, int32_t* packed_query,
                int32_t* packed_key, int32_t* routes, int32_t* lengths, void* workspace,
                hipStream_t stream, uint32_t* sign_words = nullptr, uint8_t* routed = nullptr,
                bool words_given = false) {
  Layout L = view.L;
  const ForwardWorkspace w = carve_forward(view);
  stage_begin(kStageForward, stream);
  launch_prepare_sequences(p, L, workspace, w.seq_start, w.seq_len, w.block_prefix, w.header,
                           stream);
  const int64_t elements = view.symbol_rows * L.D;
  if (words_given) {
    // a producer (the projection in front of the operator) has written the symbol words
  } else if (64 % L.D == 0) {
    hipLaunchKernelGGL(pack_symbols_ballot_kernel<DTYPE>, dim3(blocks_for(elements, 256)),
                       dim3(256), 0, stream, query, key, packed_query, packed_key, elements, L.D,
                       L.H, L.T, L.N, L.varlen);
  } else {
    hipLaunchKernelGGL(pack_symbols_rows_kernel<DTYPE>, dim3(blocks_for(view.symbol_rows, 256)),
                       dim3(256), 0, stream, query, key, packed_query, packed_key,
                       view.symbol_rows, L.D, L.H, L.T, L.N, L.varlen);
  }
  const int longest = L.varlen ? L.N : L.T;
  int shift = 1;
  while ((1 << shift) <= longest) ++shift;  // routes and runs are <= longest < 2^shift
  const bool wide = 2 * shift > 32;
  const unsigned units = static_cast<unsigned>(L.slots) * static_cast<unsigned>(L.H);
  int32_t* source_token = at<int32_t>(workspace, w.source_token);
  const uint32_t* pq = reinterpret_cast<const uint32_t*>(packed_query);
  const uint32_t* pk = reinterpret_cast<const uint32_t*>(packed_key);
  if (L.varlen) {
    if (wide) {
      hipLaunchKernelGGL((hard_route_kernel<true, true>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift);
    } else {
      hipLaunchKernelGGL((hard_route_kernel<true, false>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift);
    }
  } else {
    if (wide) {
      hipLaunchKernelGGL((hard_route_kernel<false, true>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift);
    } else {
      hipLaunchKernelGGL((hard_route_kernel<false, false>), dim3(units), dim3(kWave), 0, stream,
                         L, pq, pk, routes, lengths, source_token, shift);
    }
  }
  const int32_t* offset_error = L.varlen ? at<const int32_t>(workspace, w.header) : nullptr;
  if (sign_words != nullptr) {  // the output as sign and validity bits
    const int nvw = value_words(L.Dv);
    const int64_t words = view.symbol_rows * nvw;
    hipLaunchKernelGGL(gather_value_bits_kernel<DTYPE>, dim3(blocks_for(words, 256)), dim3(256),
                       0, stream, source_token, value, sign_words, routed, words, L.H, L.Hv,
                       L.Dv, nvw, L.T, L.N, L.varlen, offset_error);
  } else {
    const int64_t out_elements = view.symbol_rows * L.Dv;
    hipLaunchKernelGGL(gather_values_kernel<DTYPE>, dim3(blocks_for(out_elements, 256)),
                       dim3(256), 0, stream, source_token, value, output, out_elements, L.H,
                       L.Hv, L.Dv, L.T, L.N, L.varlen, offset_error);
  }
  stage_end(kStageForward, stream);
  const hipError_t status = hipGetLastError();
  if (status != hipSuccess) return fail_hip(status, "hard forward launch");
  return 0;
}

// bytes of the staged grad_output rows of a block of the row-statistics kernel
size_t row_stats_dynamic_lds(int grad_pitch) {
  constexpr int kBlockRows = kChunk;  // as in the kernel
  return sizeof(uint16_t) * kBlockRows * static_cast<size_t>(grad_pitch + 8);
}

template <int NVW, int DVP, int DT, bool VARLEN, bool DROPOUT>
int launch_vjp_passes(const VjpParams& P, const VjpWorkspace& w, bool analytic,
                      hipStream_t stream) {
  const unsigned units = static_cast<unsigned>(P.total_units);
  if (!analytic) {
    stage_begin(kStageRowMax, stream);
    hipLaunchKernelGGL((vjp_row_max_kernel<NVW, VARLEN>), dim3(units), dim3(kWave), 0, stream, P);
    stage_end(kStageRowMax, stream);
  }
  stage_begin(kStageRowStats, stream);
  hipLaunchKernelGGL((vjp_row_stats_kernel<NVW, DVP, VARLEN, DROPOUT>), dim3(units), dim3(kWave),
                     row_stats_dynamic_lds(P.grad_pitch), stream, P);
  {
    const int64_t rows = static_cast<int64_t>(P.L.N) * P.L.H;
    hipLaunchKernelGGL(finalize_row_records_kernel, dim3(blocks_for(rows, 256)), dim3(256), 0,
                       stream, P.stats, rows, P.null_logit);
  }
  stage_end(kStageRowStats, stream);
  constexpr int SEG = gradient_segment(DVP);
  // At most 64 KB of dynamic LDS per block: what every kernel may use without raising its
  // limit first.  (Raising it would be a configuration call per launch, and those are
  // refused while a stream is being captured into a graph.)
  static_assert((gradient_wave_floats(DVP, grad_term_pitch(kMaxGradTerms, DVP)) +
                 gradient_shared_fixed_floats(SEG, NVW, 1)) * sizeof(float) <= 64 * 1024,
                "dynamic LDS of the gradient kernel");
  const GradientBlockPlan plan =
      plan_gradient_blocks(DVP, P.L.D, NVW, P.grad_pitch, P.total_units);
  VjpParams Q = P;
  Q.wave_lds_floats = static_cast<int>(plan.wave_floats);
  Q.exchange_tile_floats = static_cast<int>(plan.tile_floats);
  Q.row_queue = plan.row_queue ? 1 : 0;
  const unsigned blocks = static_cast<unsigned>(std::max(1, w.resident_blocks / plan.waves));
  stage_begin(kStageGradients, stream);
  // both forms of the kernel (see its TERMS): the one that does not apply returns at once
  if (plan.waves == 2) {
    hipLaunchKernelGGL((vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 2, 2>), dim3(blocks),
                       dim3(kWave * 2), plan.lds_bytes, stream, Q);
    hipLaunchKernelGGL((vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 2, 3>), dim3(blocks),
                       dim3(kWave * 2), plan.lds_bytes, stream, Q);
  } else {
    hipLaunchKernelGGL((vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 2>), dim3(blocks),
                       dim3(kWave), plan.lds_bytes, stream, Q);
    hipLaunchKernelGGL((vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 3>), dim3(blocks),
                       dim3(kWave), plan.lds_bytes, stream, Q);
  }
  stage_end(kStageGradients, stream);
  return 0;
}

template <int NVW, int DVP, int DT>
int dispatch_vjp_layout(const VjpParams& P, const VjpWorkspace& w, bool analytic, bool dropout,
                        hipStream_t stream) {
  if (P.L.varlen) {
    return dropout ? launch_vjp_passes<NVW, DVP, DT, true, true>(P, w, analytic, stream)
                   : launch_vjp_passes<NVW, DVP, DT, true, false>(P, w, analytic, stream);
  }
  return dropout ? launch_vjp_passes<NVW, DVP, DT, false, true>(P, w, analytic, stream)
                 : launch_vjp_passes<NVW, DVP, DT, false, false>(P, w, analytic, stream);
}

template <int NVW, int DVP>
int dispatch_vjp(const VjpParams& P, const VjpWorkspace& w, bool analytic, bool dropout,
                 hipStream_t stream) {
  // symbol widths above 16 need two MFMA column tiles
  return P.L.D > 16 ? dispatch_vjp_layout<NVW, DVP, 2>(P, w, analytic, dropout, stream)
                    : dispatch_vjp_layout<NVW, DVP, 1>(P, w, analytic, dropout, stream);
}

// the analytic exponent reference is safe while it stays within 2^80 of the null weight
bool analytic_reference_is_safe(const Layout& L, float scale) {
  const int longest = L.varlen ? L.N : L.T;
  const float window = static_cast<float>(std::min(L.W, longest));
  const float bound = scale * kSqrtScale * (std::sqrt(1.0f + window) - 1.0f);
  return (bound - kNullScore * scale) * kLog2e < 80.0f;
}

template <int DTYPE>
int run_vjp(const rosa_problem* p, const ProblemView& view, const void* query, const void* key,
            const void* value, const void* grad_output, const int32_t* packed_query,
            const int32_t* packed_key, const int64_t* dropout_seed, float scale, float dropout_p,
            float inverse_keep, float mismatch_scale, int gradient_mask, float* grad_query,
            float* grad_key, float* grad_value, void* workspace, hipStream_t stream) {
  Layout L = view.L;
  const VjpWorkspace w = carve_vjp(view, dropout_p > 0.0f);
  launch_prepare_sequences(p, L, workspace, w.seq_start, w.seq_len, w.block_prefix, w.header,
                           stream, at<int64_t>(workspace, w.step_prefix), w.checkpoint_capacity);
  // Value widths above 64 are processed in slices of 64 dimensions, one full backward per
  // slice: the route weights do not depend on the values, dV of a slice needs only that
  // slice, and dQ / dK are linear in the utilities, i.e. they are the sum over the slices.
  const int full_width = L.Dv;
  const int64_t symbol_elements = view.symbol_rows * L.D;
  const int64_t value_elements = view.value_rows * full_width;
  float* sum_query = grad_query != nullptr && w.symbols_by_head ? at<float>(workspace, w.sums_query)
                                                                : grad_query;
  float* sum_key = grad_key != nullptr && w.symbols_by_head ? at<float>(workspace, w.sums_key)
                                                            : grad_key;
  float* sum_value = grad_value != nullptr && w.values_by_head ? at<float>(workspace, w.sums_value)
                                                               : grad_value;
  stage_begin(kStagePrepare, stream);
  for (int value_offset = 0; value_offset < full_width; value_offset += kValueSlice) {
    L.Dv = std::min(kValueSlice, full_width - value_offset);
    const int dvp = padded_value_width(L.Dv);
    const int nvw = value_words(L.Dv);
    if (value_offset > 0) stage_begin(kStagePrepare, stream);

    float4* stats = at<float4>(workspace, w.stats);
    uint16_t* grad_rows = at<uint16_t>(workspace, w.grad_rows);
    const int grad_pitch = grad_term_pitch(view.grad_terms, dvp);
    uint32_t* value_bits = at<uint32_t>(workspace, w.value_bits);
    int32_t* counter = at<int32_t>(workspace, w.header) + 1;
    const bool analytic = analytic_reference_is_safe(L, scale);

    {
      PrepareParams prepare;
      memset(&prepare, 0, sizeof(prepare));
      prepare.L = L;
      prepare.grad_output = grad_output;
      prepare.value = value;
      prepare.grad_rows = grad_rows;
      prepare.value_bits = value_bits;
      prepare.stats = stats;
      prepare.work_counter = counter;
      prepare.symbol_rows = view.symbol_rows;
      prepare.value_rows = view.value_rows;
      prepare.Dv = L.Dv;
      prepare.dvp = dvp;
      prepare.nvw = nvw;
      prepare.value_stride = full_width;
      prepare.value_offset = value_offset;
      prepare.grad_terms = view.grad_terms;
      prepare.grad_pitch = grad_pitch;
      prepare.scale = scale;
      prepare.analytic = analytic ? 1 : 0;
      prepare.ballot = (L.Dv == 8 || L.Dv == 16 || L.Dv == 32 || L.Dv == 64) ? 1 : 0;
      prepare.grad_blocks = blocks_for(view.symbol_rows * dvp, 256);
      prepare.value_blocks =
          blocks_for(prepare.ballot ? view.value_rows * L.Dv : view.value_rows, 256);
      prepare.stats_blocks = blocks_for(view.symbol_rows, 256);
      if (value_offset == 0) {  // the gradient buffers are cleared once, before the first slice
        // what the gradient kernel adds into: the tensors, or the head-major accumulators
        float* buffers[3] = {sum_query, sum_key, sum_value};
        const int64_t lengths[3] = {symbol_elements, symbol_elements, value_elements};
        int64_t largest = 0;
        for (int part = 0; part < 3; ++part) {
          prepare.fill[part] = buffers[part];
          prepare.fill_elements[part] = buffers[part] != nullptr ? lengths[part] : 0;
          largest = std::max(largest, prepare.fill_elements[part]);
        }
        prepare.fill_blocks =
            static_cast<unsigned>(std::min<int64_t>(blocks_for(largest, 256), 8192));
      }
      const unsigned blocks = prepare.grad_blocks + prepare.value_blocks + prepare.stats_blocks +
                              prepare.fill_blocks;
      if (L.varlen) {
        hipLaunchKernelGGL((vjp_prepare_kernel<DTYPE, true>), dim3(blocks), dim3(256), 0, stream,
                           prepare);
      } else {
        hipLaunchKernelGGL((vjp_prepare_kernel<DTYPE, false>), dim3(blocks), dim3(256), 0, stream,
                           prepare);
      }
    }

    stage_end(kStagePrepare, stream);

    VjpParams P;
    memset(&P, 0, sizeof(P));
    P.L = L;
    P.packed_query = reinterpret_cast<const uint32_t*>(packed_query);
    P.packed_key = reinterpret_cast<const uint32_t*>(packed_key);
    P.value_bits = value_bits;
    P.grad_rows = grad_rows;
    P.grad_terms = view.grad_terms;
    P.grad_pitch = grad_pitch;
    P.stats = stats;
    P.dropout_seed = dropout_seed;
    P.scale = scale;
    P.dropout_p = dropout_p;
    P.inverse_keep = inverse_keep;
    P.mismatch_scale = mismatch_scale;
    P.gate_log2 = mismatch_scale * kLog2e / static_cast<float>(L.D);
    P.logit_gain = scale * kSqrtScale * kLog2e;
    P.null_logit = kNullScore * scale;
    {
      // window products this far below one cannot move a float32 gradient:
      // 2^-34 / (W^2 * longest)
      const int longest = L.varlen ? L.N : L.T;
      const float exponent =
          -34.0f - 2.0f * std::log2(static_cast<float>(L.W)) -
          std::log2(static_cast<float>(longest));
      P.tail_threshold = std::exp2(std::max(exponent, -120.0f));
    }
    P.gradient_mask = gradient_mask;
    P.dvp = dvp;
    P.grad_query = sum_query;
    P.grad_key = sum_key;
    P.grad_value = sum_value;
    P.symbols_by_head = w.symbols_by_head ? 1 : 0;
    P.values_by_head = w.values_by_head ? 1 : 0;
    P.work_counter = counter;
    P.header = at<int32_t>(workspace, w.header);
    // The records hold saturated window counts: they are kept when no count can saturate, or
    // when every count that can still produce a relevant overflow term within a chunk lies
    // below the saturation value (otherwise, with a long window and a tiny mismatch_scale,
    // the gradient pass rebuilds the evidence itself).
    const bool windows_fit =
        static_cast<int64_t>(w.ring_rows) * L.D <= kRecordWindowMax ||
        -std::log2(P.tail_threshold) / P.gate_log2 + kChunk * L.D + 2 <= kRecordWindowMax;
    P.checkpoints = (w.checkpoint_capacity > 0 && windows_fit) ? at<float>(workspace, w.checkpoints)
                                                              : nullptr;
    P.record_floats = w.record_floats;
    P.value_stride = full_width;
    P.value_offset = value_offset;
    P.block_scratch = at<float>(workspace, w.block_scratch);
    P.block_scratch_floats = w.block_scratch_floats;
    P.segment_group = w.segment_group;
    P.ring_rows = w.ring_rows;
    P.total_units = L.slots * L.H;
    const bool dropout = dropout_p > 0.0f;

    int status = 0;
    if (nvw == 1) {
      if (dvp == 8) status = dispatch_vjp<1, 8>(P, w, analytic, dropout, stream);
      else if (dvp == 16) status = dispatch_vjp<1, 16>(P, w, analytic, dropout, stream);
      else status = dispatch_vjp<1, 32>(P, w, analytic, dropout, stream);
    } else {
      status = dispatch_vjp<2, 64>(P, w, analytic, dropout, stream);
    }
    if (status != 0) return status;
  }  // value slices
  const int64_t finalize_items = std::max(symbol_elements, value_elements);
  stage_begin(kStageFinalize, stream);
  HeadMajorSums sums;
  sums.query = sum_query != grad_query ? sum_query : nullptr;
  sums.key = sum_key != grad_key ? sum_key : nullptr;
  sums.value = sum_value != grad_value ? sum_value : nullptr;
  sums.H = L.H; sums.Hv = L.Hv; sums.D = L.D; sums.Dv = full_width;
  sums.T = L.T; sums.N = L.N; sums.varlen = L.varlen ? 1 : 0;
  hipLaunchKernelGGL(finalize_gradients_kernel<DTYPE>, dim3(blocks_for(finalize_items, 256)),
                     dim3(256), 0, stream, query, key, value, grad_query, grad_key, grad_value,
                     symbol_elements, value_elements,
                     L.varlen ? at<const int32_t>(workspace, w.header) : nullptr, sums);
  stage_end(kStageFinalize, stream);
  const hipError_t launch = hipGetLastError();
  if (launch != hipSuccess) return fail_hip(launch, "surrogate vjp launch");
  return 0;
}


// ---------------------------------------------------------------------------
// streaming hard router (inference): the hard forward over a growing history
// ---------------------------------------------------------------------------
//
// Every (slot, head) keeps its query, key and payload symbols (one byte each) in
// device memory, `capacity` bytes per run.  An update appends a chunk of tokens to
// every slot and routes exactly the new rows against all keys before them; the
// answer per row is the end position of the matched key (route - 1, or -1 for the
// null route) and the payload symbol that follows it.

constexpr int kRouterDecodeRows = 8;  // chunks up to this many rows use the per-row kernel

struct RouterUpdate {
  int S, H, Hp, W;
  int capacity;
  int qk_mask, payload_mask;
  const int32_t* chunk_offsets;  // [S + 1] token offsets of the chunk per slot, or NULL:
  int uniform_chunk;             //   then every slot brings this many tokens
  int32_t* history_lengths;      // [S] tokens a slot held before this chunk (advanced at the end)
  uint8_t* query_history;        // [S][H][capacity]
  uint8_t* key_history;          // [S][H][capacity]
  uint8_t* payload_history;      // [S][Hp][capacity]
  const uint8_t* query;          // [tokens][H]
  const uint8_t* key;            // [tokens][H]
  const uint8_t* payload;        // [tokens][Hp]
  uint8_t* output;               // [tokens][H]
  int64_t* matched_key_end;      // [tokens][H]
  int tokens;
  int blocks_per_run;            // blocks of the routing grid that share one (slot, head)
};

__device__ __forceinline__ int router_chunk_begin(const RouterUpdate& U, int slot) {
  return U.chunk_offsets != nullptr ? U.chunk_offsets[slot] : slot * U.uniform_chunk;
}

__global__ __launch_bounds__(256) void router_append_kernel(RouterUpdate U) {
  const int64_t index = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (index >= static_cast<int64_t>(U.tokens) * U.H) return;
  const int token = static_cast<int>(index / U.H);
  const int head = static_cast<int>(index - static_cast<int64_t>(token) * U.H);
  int slot;
  if (U.chunk_offsets == nullptr) {
    slot = token / U.uniform_chunk;
  } else {
    int low = 0, high = U.S;  // last slot with offsets[slot] <= token (empty slots share offsets)
    while (low + 1 < high) {
      const int mid = (low + high) >> 1;
      if (U.chunk_offsets[mid] <= token) low = mid; else high = mid;
    }
    slot = low;
  }
  const int position = U.history_lengths[slot] + (token - router_chunk_begin(U, slot));
  const int64_t run = (static_cast<int64_t>(slot) * U.H + head) * U.capacity + position;
  U.query_history[run] = U.query[index] & U.qk_mask;
  U.key_history[run] = U.key[index] & U.qk_mask;
  if (head < U.Hp) {
    U.payload_history[(static_cast<int64_t>(slot) * U.Hp + head) * U.capacity + position] =
        U.payload[static_cast<int64_t>(token) * U.Hp + head] & U.payload_mask;
  }
}

// One wave owns 64 consecutive new rows of one (slot, head) (lane = row) and walks over
// the routes exactly like hard_route_kernel; the first row block starts at the slot's old
// length, so its predecessor row lies in the history.
__global__ __launch_bounds__(kWave) void router_route_kernel(RouterUpdate U) {
  // one-dimensional grid: (slot, head) run-major, so that slots * heads is not bounded by
  // the 65535 blocks of the other grid dimensions
  const int run = static_cast<int>(blockIdx.x / static_cast<unsigned>(U.blocks_per_run));
  const int row_block = static_cast<int>(blockIdx.x - static_cast<unsigned>(run) * U.blocks_per_run);
  const int slot = run / U.H;
  const int head = run - slot * U.H;
  const int old_length = U.history_lengths[slot];
  const int chunk_begin = router_chunk_begin(U, slot);
  const int new_length = old_length + (router_chunk_begin(U, slot + 1) - chunk_begin);
  const int t0 = old_length + row_block * kWave;
  if (t0 >= new_length) return;
  const int lane = threadIdx.x;
  const int64_t run_base = (static_cast<int64_t>(slot) * U.H + head) * U.capacity;
  const uint8_t* q = U.query_history + run_base;
  const uint8_t* k = U.key_history + run_base;
  const int t = t0 + lane;
  const bool row_ok = t < new_length;
  const uint32_t q_symbol = row_ok ? q[t] : 0u;
  const int shift = 32 - __clz(new_length);  // new_length < 2^shift
  const bool narrow = shift <= 16 && U.W < 65536;
  const RouteWinner winner =
      narrow ? scan_routes_narrow(q, k, t0, new_length, U.W, shift, lane, q_symbol)
             : scan_routes_wide(q, k, t0, new_length, U.W, lane, q_symbol);
  if (!row_ok) return;
  const int route = winner.run > 0 ? winner.route : 0;
  const int64_t token = chunk_begin + (t - old_length);
  const int payload_head = head / (U.H / U.Hp);
  U.matched_key_end[token * U.H + head] = route > 0 ? route - 1 : -1;
  U.output[token * U.H + head] = route > 0
      ? U.payload_history[(static_cast<int64_t>(slot) * U.Hp + payload_head) * U.capacity + route]
      : uint8_t(0);
}


// Few new rows per slot (decoding): one wave per (slot, head, new row); the lanes share the
// routes of the row, each comparing its suffixes directly, and the wave keeps the maximum of
// the packed key (length, route): longest first, latest on ties.
__global__ __launch_bounds__(kWave) void router_decode_kernel(RouterUpdate U) {
  const int run = static_cast<int>(blockIdx.x / static_cast<unsigned>(U.blocks_per_run));
  const int row = static_cast<int>(blockIdx.x - static_cast<unsigned>(run) * U.blocks_per_run);
  const int slot = run / U.H;
  const int head = run - slot * U.H;
  const int old_length = U.history_lengths[slot];
  const int chunk_begin = router_chunk_begin(U, slot);
  const int rows = router_chunk_begin(U, slot + 1) - chunk_begin;
  if (row >= rows) return;
  const int lane = threadIdx.x;
  const int t = old_length + row;
  const int64_t run_base = (static_cast<int64_t>(slot) * U.H + head) * U.capacity;
  const uint8_t* q = U.query_history + run_base;
  const uint8_t* k = U.key_history + run_base;
  unsigned long long best = 0ull;
  for (int a = 1 + lane; a <= t; a += kWave) {
    const int limit = min(U.W, a);
    int length = 0;
    while (length < limit && q[t - length] == k[a - 1 - length]) ++length;
    const unsigned long long packed =
        (static_cast<unsigned long long>(length) << 32) | static_cast<uint32_t>(a);
    best = max(best, packed);
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    best = max(best, static_cast<unsigned long long>(__shfl_xor(best, offset, kWave)));
  }
  if (lane != 0) return;
  const int route = (best >> 32) > 0 ? static_cast<int>(best & 0xffffffffull) : 0;
  const int64_t token = chunk_begin + row;
  const int payload_head = head / (U.H / U.Hp);
  U.matched_key_end[token * U.H + head] = route > 0 ? route - 1 : -1;
  U.output[token * U.H + head] = route > 0
      ? U.payload_history[(static_cast<int64_t>(slot) * U.Hp + payload_head) * U.capacity + route]
      : uint8_t(0);
}

__global__ __launch_bounds__(256) void router_advance_kernel(RouterUpdate U) {
  const int slot = blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= U.S) return;
  U.history_lengths[slot] += router_chunk_begin(U, slot + 1) - router_chunk_begin(U, slot);
}

// ---------------------------------------------------------------------------
// the projection that follows the operator, fed with the bit form of its output
// ---------------------------------------------------------------------------
//
//   out[t, n] = residual[t, n] + sum_k y[t, k] * weight[n, k],   k = h * Dv + d,
//   y[t, k] = routed[t, h] ? (bit d of sign_words[t, h] ? +1 : -1) : 0
//
// i.e. `residual + output(routed.flatten(2))` of the reference's caller
// (examples/fit_soft_reference.py:374-417) without the ternary tensor in between: the A
// operand of the matrix products is expanded from the bits in registers.  `weight` is the
// [N][K] matrix of a linear layer (k contiguous), bfloat16; accumulation is float32.
// A block of four waves computes 256 rows x 64 columns, each wave 64 x 64 (sixteen
// 16 x 16 x 32 products per 32-wide k step).  Per step a block stages the weight tile
// [64][32] and, per row, the 32 sign bits and 32 validity bits of the step in LDS; the loads
// of the next step are in flight while the products of this one run.
constexpr int kProjectRows = 256;
constexpr int kProjectColumns = 64;
constexpr int kProjectStep = 32;
constexpr int kProjectWeightPitch = kProjectStep + 8;  // bfloat16 elements per staged weight row

struct ProjectParams {
  const uint32_t* sign_words;  // [tokens][H][nvw]
  const uint8_t* routed;       // [tokens][H]
  const uint16_t* weight;      // [N][K] bfloat16
  const uint16_t* residual;    // [tokens][N] bfloat16 or NULL
  uint16_t* out;               // [tokens][N] bfloat16
  int64_t tokens;
  int H, Dv, nvw, N, K;
};

// Eight sign bits and their validity -> eight bfloat16 values (two table entries of four):
// entry (valid << 4 | nibble) holds +-1 per bit, or zeros where the head took the null route.
constexpr int kTernaryTableWords = 64;

__device__ __forceinline__ void fill_ternary_table(uint32_t* table, int index) {
  if (index < kTernaryTableWords) {
    const int entry = index >> 1;       // valid << 4 | nibble
    const int nibble = entry & 15;
    const bool valid = (entry >> 4) != 0;
    const int low = (nibble >> (2 * (index & 1))) & 1;
    const int high = (nibble >> (2 * (index & 1) + 1)) & 1;
    table[index] = valid ? ((low ? 0x3f80u : 0xbf80u) | ((high ? 0x3f80u : 0xbf80u) << 16)) : 0u;
  }
}

// sign bits and validity bits of k = 32 step .. 32 step + 31 of one token
__device__ __forceinline__ uint2 ternary_step_bits(const ProjectParams& P, int64_t token, int step) {
  const int k0 = step * kProjectStep;
  uint32_t signs = 0u, valid = 0u;
  if (token < P.tokens) {
    if (P.Dv >= 32) {  // the step lies inside one head
      const int head = k0 / P.Dv;
      const int word = (k0 - head * P.Dv) >> 5;
      signs = P.sign_words[(token * P.H + head) * P.nvw + word];
      valid = P.routed[token * P.H + head] == 1 ? 0xffffffffu : 0u;
    } else {           // 32 / Dv heads, one word each
      const int heads = 32 / P.Dv;
      const int head0 = k0 / P.Dv;
      const uint32_t field = (1u << P.Dv) - 1u;
      for (int j = 0; j < heads; ++j) {
        const uint32_t word = P.sign_words[token * P.H + head0 + j] & field;
        signs |= word << (j * P.Dv);
        if (P.routed[token * P.H + head0 + j] == 1) valid |= field << (j * P.Dv);
      }
    }
  }
  return make_uint2(signs, valid);
}

__global__ __launch_bounds__(256) void project_routed_bits_kernel(ProjectParams P) {
  __shared__ __attribute__((aligned(16))) uint16_t weight_tile[2][kProjectColumns * kProjectWeightPitch];
  __shared__ __attribute__((aligned(8))) uint2 row_bits[2][kProjectRows];
  __shared__ __attribute__((aligned(8))) uint32_t ternary_table[kTernaryTableWords];
  const int thread = threadIdx.x;
  const int lane = thread & 63;
  const int wave = thread >> 6;
  const int li = lane & 15;
  const int lg = lane >> 4;
  // neighbouring blocks share their weight columns (same blockIdx.y) and follow each other
  // in row order, so the weight tiles of a column block stay in the cache of their XCD
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kProjectRows;
  const int n0 = blockIdx.y * kProjectColumns;
  fill_ternary_table(ternary_table, thread);

  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  }
  const int steps = P.K / kProjectStep;
  // what a thread stages per step: 16 bytes of the weight tile and one row's bits
  const int stage_n = thread >> 2;
  const int stage_k = (thread & 3) * 8;
  const uint16_t* weight_row = P.weight + static_cast<int64_t>(n0 + stage_n) * P.K + stage_k;
  uint4 weight_in = *reinterpret_cast<const uint4*>(weight_row);
  uint2 bits_in = ternary_step_bits(P, row0 + thread, 0);
  for (int step = 0; step < steps; ++step) {
    const int buffer = step & 1;
    *reinterpret_cast<uint4*>(&weight_tile[buffer][stage_n * kProjectWeightPitch + stage_k]) = weight_in;
    row_bits[buffer][thread] = bits_in;
    __syncthreads();
    if (step + 1 < steps) {  // the next step's loads are in flight during the products
      weight_in = *reinterpret_cast<const uint4*>(weight_row + (step + 1) * kProjectStep);
      bits_in = ternary_step_bits(P, row0 + thread, step + 1);
    }
    v4u b_operand[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      b_operand[j] = *reinterpret_cast<const v4u*>(
          &weight_tile[buffer][(16 * j + li) * kProjectWeightPitch + 8 * lg]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint2 bits = row_bits[buffer][wave * 64 + 16 * i + li];
      const uint32_t byte = (bits.x >> (8 * lg)) & 0xffu;
      const uint32_t valid = (bits.y >> (8 * lg)) & 1u;  // a head is valid as a whole
      const uint2 low = *reinterpret_cast<const uint2*>(
          ternary_table + 2 * ((valid << 4) | (byte & 15u)));
      const uint2 high = *reinterpret_cast<const uint2*>(
          ternary_table + 2 * ((valid << 4) | (byte >> 4)));
      const v4u a_operand = {low.x, low.y, high.x, high.y};
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = mfma_bf16(a_operand, b_operand[j], acc[i][j]);
    }
  }
  // lane (li, lg) holds rows 4 lg .. 4 lg + 3 of column li of every 16 x 16 tile
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t token = row0 + wave * 64 + 16 * i + 4 * lg + e;
      if (token >= P.tokens) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t index = token * P.N + n0 + 16 * j + li;
        float value = acc[i][j][e];
        if (P.residual != nullptr) value += __uint_as_float(static_cast<uint32_t>(P.residual[index]) << 16);
        P.out[index] = static_cast<uint16_t>(bf16_nearest(value));
      }
    }
  }
}

int forward_entry(const rosa_problem* problem, const void* query, const void* key,
                  const void* value, void* output, int32_t* packed_query, int32_t* packed_key,
                  int32_t* routes, int32_t* lengths, void* workspace, size_t workspace_bytes,
                  void* stream, uint32_t* sign_words, uint8_t* routed, bool words_given = false) {
  ProblemView view;
  const int bad = check_problem(problem, &view);
  if (bad != 0) return bad;
  if ((!words_given && (!query || !key)) || !value || !packed_query || !packed_key || !workspace)
    return fail(2, "hard_forward: NULL tensor or workspace pointer");
  if (workspace_bytes < carve_forward(view).total) return fail(3, "hard_forward: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (problem->dtype) {
    case ROSA_DTYPE_F32:
      return run_forward<ROSA_DTYPE_F32>(problem, view, query, key, value, output, packed_query,
                                         packed_key, routes, lengths, workspace, s, sign_words,
                                         routed, words_given);
    case ROSA_DTYPE_F16:
      return run_forward<ROSA_DTYPE_F16>(problem, view, query, key, value, output, packed_query,
                                         packed_key, routes, lengths, workspace, s, sign_words,
                                         routed, words_given);
    default:
      return run_forward<ROSA_DTYPE_BF16>(problem, view, query, key, value, output, packed_query,
                                          packed_key, routes, lengths, workspace, s, sign_words,
                                          routed, words_given);
  }
}

// Address of the current device's copy of `scratch`, looked up once per device.
constexpr int kMaxDevices = 64;
void* g_scratch_address[kMaxDevices];
std::mutex g_scratch_mutex;

int static_scratch_address(void** address) {
  int device = -1;
  const hipError_t current = hipGetDevice(&device);
  if (current != hipSuccess) return fail_hip(current, "hipGetDevice");
  if (device < 0 || device >= kMaxDevices) return fail(4, "static scratch: device index out of range");
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (g_scratch_address[device] == nullptr) {
    void* found = nullptr;
    const hipError_t status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return fail_hip(status, "hipGetSymbolAddress(scratch)");
    if (found == nullptr) return fail(4, "static scratch: no device address");
    g_scratch_address[device] = found;
  }
  *address = g_scratch_address[device];
  return 0;
}

template <int DTYPE>
void launch_pack_rows(const void* logits, int64_t rows, int bits, void* symbols, int symbol_bytes,
                      hipStream_t stream) {
  const int64_t elements = rows * bits;
  if (64 % bits == 0) {
    const dim3 grid(blocks_for(elements, 256));
    if (symbol_bytes == 1) {
      hipLaunchKernelGGL((pack_rows_ballot_kernel<DTYPE, uint8_t>), grid, dim3(256), 0, stream,
                         logits, static_cast<uint8_t*>(symbols), elements, bits);
    } else {
      hipLaunchKernelGGL((pack_rows_ballot_kernel<DTYPE, uint32_t>), grid, dim3(256), 0, stream,
                         logits, static_cast<uint32_t*>(symbols), elements, bits);
    }
  } else {
    const dim3 grid(blocks_for(rows, 256));
    if (symbol_bytes == 1) {
      hipLaunchKernelGGL((pack_rows_serial_kernel<DTYPE, uint8_t>), grid, dim3(256), 0, stream,
                         logits, static_cast<uint8_t*>(symbols), rows, bits);
    } else {
      hipLaunchKernelGGL((pack_rows_serial_kernel<DTYPE, uint32_t>), grid, dim3(256), 0, stream,
                         logits, static_cast<uint32_t*>(symbols), rows, bits);
    }
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------

extern "C" {

int rosa_hip_version(void) { return 100; }

const char* rosa_hip_target(void) { return "rocm-gfx950"; }

const char* rosa_hip_last_error(void) { return g_error; }

size_t rosa_hip_forward_workspace_bytes(const rosa_problem* problem) {
  ProblemView view;
  if (check_problem(problem, &view) != 0) return 0;
  return carve_forward(view).total;
}

size_t rosa_hip_vjp_workspace_bytes(const rosa_problem* problem, int gradient_mask, float scale,
                                    int dropout) {
  (void)gradient_mask;
  (void)scale;
  ProblemView view;
  if (check_problem(problem, &view) != 0) return 0;
  return carve_vjp(view, dropout != 0).total;
}

int rosa_hip_hard_routes(const rosa_problem* problem, const void* query, const void* key,
                         const void* value, void* output, int32_t* packed_query,
                         int32_t* packed_key, int32_t* routes, int32_t* lengths,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (!output) return fail(2, "hard_forward: NULL tensor or workspace pointer");
  return forward_entry(problem, query, key, value, output, packed_query, packed_key, routes,
                       lengths, workspace, workspace_bytes, stream, nullptr, nullptr);
}

int rosa_hip_hard_forward_bits(const rosa_problem* problem, const void* query, const void* key,
                               const void* value, uint32_t* sign_words, uint8_t* routed,
                               int32_t* packed_query, int32_t* packed_key, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (!sign_words || !routed) return fail(2, "hard_forward_bits: NULL output pointer");
  return forward_entry(problem, query, key, value, nullptr, packed_query, packed_key, nullptr,
                       nullptr, workspace, workspace_bytes, stream, sign_words, routed);
}

int rosa_hip_hard_forward_words(const rosa_problem* problem, const int32_t* packed_query,
                                const int32_t* packed_key, const void* value, void* output,
                                uint32_t* sign_words, uint8_t* routed, int32_t* routes,
                                void* workspace, size_t workspace_bytes, void* stream) {
  if (!output && !(sign_words && routed))
    return fail(2, "hard_forward_words: give the output tensor or both parts of its bit form");
  if (output) { sign_words = nullptr; routed = nullptr; }
  return forward_entry(problem, nullptr, nullptr, value, output, const_cast<int32_t*>(packed_query),
                       const_cast<int32_t*>(packed_key), routes, nullptr, workspace,
                       workspace_bytes, stream, sign_words, routed, true);
}

int rosa_hip_project_routed_bits(const uint32_t* sign_words, const uint8_t* routed,
                                 int64_t tokens, int H, int Dv, const void* weight, int N,
                                 const void* residual, void* out, void* stream) {
  if (tokens < 0 || H < 1 || Dv < 1 || N < 1) return fail(1, "project_routed_bits: bad sizes");
  if (tokens == 0) return 0;
  if (!sign_words || !routed || !weight || !out) return fail(2, "project_routed_bits: NULL pointer");
  const int64_t K = static_cast<int64_t>(H) * Dv;
  if (Dv % 8 != 0 || !(32 % Dv == 0 || Dv % 32 == 0) || K % kProjectStep != 0 || K > INT32_MAX)
    return fail(1, "project_routed_bits: the value width must be 8, 16 or a multiple of 32, and "
                   "H * Dv a multiple of 32");
  if (N % kProjectColumns != 0)
    return fail(1, "project_routed_bits: the output width must be a multiple of 64");
  const int64_t row_blocks = (tokens + kProjectRows - 1) / kProjectRows;
  if (row_blocks > INT32_MAX || N / kProjectColumns > 65535)
    return fail(1, "project_routed_bits: too many blocks");
  ProjectParams P;
  P.sign_words = sign_words;
  P.routed = routed;
  P.weight = static_cast<const uint16_t*>(weight);
  P.residual = static_cast<const uint16_t*>(residual);
  P.out = static_cast<uint16_t*>(out);
  P.tokens = tokens;
  P.H = H; P.Dv = Dv; P.nvw = value_words(Dv); P.N = N; P.K = static_cast<int>(K);
  hipLaunchKernelGGL(project_routed_bits_kernel,
                     dim3(static_cast<unsigned>(row_blocks), static_cast<unsigned>(N / kProjectColumns)),
                     dim3(256), 0, static_cast<hipStream_t>(stream), P);
  const hipError_t launch = hipGetLastError();
  if (launch != hipSuccess) return fail_hip(launch, "project_routed_bits launch");
  return 0;
}

int rosa_hip_hard_forward_static(const rosa_problem* problem, const void* query, const void* key,
                                 const void* value, void* output, int32_t* packed_query,
                                 int32_t* packed_key, int32_t* routes, void* stream) {
  if (!output) return fail(2, "hard_forward_static: NULL tensor pointer");
  ProblemView view;
  const int bad = check_problem(problem, &view);
  if (bad != 0) return bad;
  if (carve_forward(view).total > kStaticScratchBytes) {
    return fail(3, "hard_forward_static: the problem needs more than the 16 MiB of static "
                   "scratch (4 bytes per token and head); use rosa_hip_hard_forward");
  }
  void* address = nullptr;
  const int status = static_scratch_address(&address);
  if (status != 0) return status;
  return forward_entry(problem, query, key, value, output, packed_query, packed_key, routes,
                       nullptr, address, kStaticScratchBytes, stream, nullptr, nullptr);
}

int rosa_hip_pack_symbols(int dtype, const void* logits, int64_t rows, int bits, void* symbols,
                          int symbol_bytes, void* stream) {
  if (dtype < ROSA_DTYPE_F32 || dtype > ROSA_DTYPE_BF16) return fail(1, "unsupported dtype");
  if (rows < 0) return fail(1, "pack_symbols: negative row count");
  if (symbol_bytes != 1 && symbol_bytes != 4)
    return fail(1, "pack_symbols: symbols are stored as 1 or 4 bytes");
  if (bits < 1 || bits > 8 * symbol_bytes)
    return fail(1, "pack_symbols: symbol width must be in [1, 8] for bytes and [1, 32] for words");
  if (rows == 0) return 0;
  if (!logits || !symbols) return fail(2, "pack_symbols: NULL pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case ROSA_DTYPE_F32:
      launch_pack_rows<ROSA_DTYPE_F32>(logits, rows, bits, symbols, symbol_bytes, s);
      break;
    case ROSA_DTYPE_F16:
      launch_pack_rows<ROSA_DTYPE_F16>(logits, rows, bits, symbols, symbol_bytes, s);
      break;
    default:
      launch_pack_rows<ROSA_DTYPE_BF16>(logits, rows, bits, symbols, symbol_bytes, s);
  }
  const hipError_t launch = hipGetLastError();
  if (launch != hipSuccess) return fail_hip(launch, "pack_symbols launch");
  return 0;
}

int rosa_hip_hard_forward(const rosa_problem* problem, const void* query, const void* key,
                          const void* value, void* output, int32_t* packed_query,
                          int32_t* packed_key, int32_t* routes, void* workspace,
                          size_t workspace_bytes, void* stream) {
  return rosa_hip_hard_routes(problem, query, key, value, output, packed_query, packed_key,
                              routes, nullptr, workspace, workspace_bytes, stream);
}

int rosa_hip_surrogate_vjp(const rosa_problem* problem, const void* query, const void* key,
                           const void* value, const void* grad_output,
                           const int32_t* packed_query, const int32_t* packed_key,
                           const int64_t* dropout_seed, float scale, float dropout_p,
                           float inverse_keep, float mismatch_scale, int gradient_mask,
                           float* grad_query, float* grad_key, float* grad_value, void* workspace,
                           size_t workspace_bytes, void* stream) {
  ProblemView view;
  const int bad = check_problem(problem, &view);
  if (bad != 0) return bad;
  if (gradient_mask < 1 || gradient_mask > 7)
    return fail(1, "gradient_mask must be an integer bit mask in [1, 7]");
  if (!query || !key || !value || !grad_output || !packed_query || !packed_key || !workspace)
    return fail(2, "surrogate_vjp: NULL tensor or workspace pointer");
  if (((gradient_mask & ROSA_GRAD_QUERY) && !grad_query) ||
      ((gradient_mask & ROSA_GRAD_KEY) && !grad_key) ||
      ((gradient_mask & ROSA_GRAD_VALUE) && !grad_value))
    return fail(2, "surrogate_vjp: a requested gradient has a NULL pointer");
  if (!(scale > 0.0f) || !(mismatch_scale > 0.0f) || !(dropout_p >= 0.0f) || !(dropout_p < 1.0f))
    return fail(1, "surrogate_vjp: scale, mismatch_scale > 0 and 0 <= dropout_p < 1 required");
  if (dropout_p > 0.0f && dropout_seed == nullptr)
    return fail(2, "surrogate_vjp: dropout_seed must be given exactly when dropout_p > 0");
  if (workspace_bytes < carve_vjp(view, dropout_p > 0.0f).total)
    return fail(3, "surrogate_vjp: workspace too small");
  if (!(gradient_mask & ROSA_GRAD_QUERY)) grad_query = nullptr;
  if (!(gradient_mask & ROSA_GRAD_KEY)) grad_key = nullptr;
  if (!(gradient_mask & ROSA_GRAD_VALUE)) grad_value = nullptr;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (problem->dtype) {
    case ROSA_DTYPE_F32:
      return run_vjp<ROSA_DTYPE_F32>(problem, view, query, key, value, grad_output, packed_query,
                                     packed_key, dropout_seed, scale, dropout_p, inverse_keep,
                                     mismatch_scale, gradient_mask, grad_query, grad_key,
                                     grad_value, workspace, s);
    case ROSA_DTYPE_F16:
      return run_vjp<ROSA_DTYPE_F16>(problem, view, query, key, value, grad_output, packed_query,
                                     packed_key, dropout_seed, scale, dropout_p, inverse_keep,
                                     mismatch_scale, gradient_mask, grad_query, grad_key,
                                     grad_value, workspace, s);
    default:
      return run_vjp<ROSA_DTYPE_BF16>(problem, view, query, key, value, grad_output, packed_query,
                                      packed_key, dropout_seed, scale, dropout_p, inverse_keep,
                                      mismatch_scale, gradient_mask, grad_query, grad_key,
                                      grad_value, workspace, s);
  }
}

int rosa_hip_router_update(const rosa_router_update* update, void* stream) {
  if (update == nullptr) return fail(1, "router update is NULL");
  const rosa_router_update& u = *update;
  if (u.S < 1 || u.H < 1 || u.Hp < 1 || u.H % u.Hp != 0)
    return fail(1, "router: heads must be a positive multiple of payload heads");
  if (u.qk_bits < 1 || u.qk_bits > 8 || u.payload_bits < 1 || u.payload_bits > 8)
    return fail(1, "router: symbol widths must be in [1, 8]");
  if (u.W < 1) return fail(1, "router: max_suffix_length must be >= 1");
  if (u.tokens < 0 || u.longest_chunk < 0 || u.capacity < 1)
    return fail(1, "router: negative size");
  if (u.tokens == 0) return 0;
  if (!u.chunk_offsets && static_cast<int64_t>(u.uniform_chunk) * u.S != u.tokens)
    return fail(1, "router: without chunk_offsets every slot brings uniform_chunk tokens");
  if (!u.history_lengths || !u.query_history || !u.key_history ||
      !u.payload_history || !u.query || !u.key || !u.payload || !u.output || !u.matched_key_end)
    return fail(2, "router: NULL pointer");
  RouterUpdate U;
  U.S = u.S; U.H = u.H; U.Hp = u.Hp; U.W = u.W;
  U.capacity = u.capacity;
  U.qk_mask = (1 << u.qk_bits) - 1;
  U.payload_mask = (1 << u.payload_bits) - 1;
  U.chunk_offsets = u.chunk_offsets;
  U.uniform_chunk = u.uniform_chunk;
  U.history_lengths = u.history_lengths;
  U.query_history = u.query_history;
  U.key_history = u.key_history;
  U.payload_history = u.payload_history;
  U.query = u.query; U.key = u.key; U.payload = u.payload;
  U.output = u.output;
  U.matched_key_end = u.matched_key_end;
  U.tokens = u.tokens;
  U.blocks_per_run = 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t symbols = static_cast<int64_t>(u.tokens) * u.H;
  hipLaunchKernelGGL(router_append_kernel, dim3(blocks_for(symbols, 256)), dim3(256), 0, s, U);
  const int64_t runs = static_cast<int64_t>(u.S) * u.H;
  if (u.longest_chunk > 0) {
    const bool decode = u.longest_chunk <= kRouterDecodeRows;
    U.blocks_per_run = decode ? u.longest_chunk : (u.longest_chunk + kWave - 1) / kWave;
    const int64_t blocks = runs * U.blocks_per_run;
    if (blocks > INT32_MAX) return fail(1, "router: slots * heads * row blocks must fit in int32");
    if (decode) {
      hipLaunchKernelGGL(router_decode_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWave), 0,
                         s, U);
    } else {
      hipLaunchKernelGGL(router_route_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWave), 0,
                         s, U);
    }
  }
  hipLaunchKernelGGL(router_advance_kernel, dim3(blocks_for(u.S, 256)), dim3(256), 0, s, U);
  const hipError_t status = hipGetLastError();
  if (status != hipSuccess) return fail_hip(status, "router launch");
  return 0;
}

void rosa_hip_set_gradient_block_waves(int waves) {
  g_gradient_block_waves = (waves == 1 || waves == 2) ? waves : 0;
}

void rosa_hip_set_record_budget(size_t bytes) {
  g_record_budget_bytes = bytes;  // (size_t)-1: the default
}

int rosa_hip_stage_timing(int enable) {
  if (enable && !g_timer.created) {
    for (int i = 0; i < kStageCount; ++i) {
      if (hipEventCreate(&g_timer.begin[i]) != hipSuccess) return fail(5, "hipEventCreate failed");
      if (hipEventCreate(&g_timer.end[i]) != hipSuccess) return fail(5, "hipEventCreate failed");
    }
    g_timer.created = true;
  }
  for (int i = 0; i < kStageCount; ++i) g_timer.used[i] = false;
  g_timer.enabled = enable != 0;
  return 0;
}

int rosa_hip_stage_count(void) { return kStageCount; }

const char* rosa_hip_stage_name(int stage) {
  static const char* names[kStageCount] = {"hard_forward", "vjp_prepare", "vjp_row_max",
                                           "vjp_row_stats", "vjp_gradients", "vjp_finalize"};
  return (stage >= 0 && stage < kStageCount) ? names[stage] : "";
}

int rosa_hip_stage_times(float* milliseconds, int count) {
  if (!g_timer.created) return fail(5, "stage timing was never enabled");
  for (int i = 0; i < count && i < kStageCount; ++i) {
    milliseconds[i] = -1.0f;
    if (!g_timer.used[i]) continue;
    if (hipEventSynchronize(g_timer.end[i]) != hipSuccess) return fail(5, "event sync failed");
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, g_timer.begin[i], g_timer.end[i]) != hipSuccess)
      return fail(5, "event elapsed failed");
    milliseconds[i] = ms;
  }
  return 0;
}

int rosa_hip_gradient_block_plan(const rosa_problem* problem, int* waves, int* row_queue,
                                 size_t* lds_bytes) {
  ProblemView view;
  const int status = check_problem(problem, &view);
  if (status != 0) return status;
  const int slice_width = std::min(view.L.Dv, kValueSlice);
  const int dvp = padded_value_width(slice_width);
  const GradientBlockPlan plan =
      plan_gradient_blocks(dvp, view.L.D, value_words(slice_width),
                           grad_term_pitch(view.grad_terms, dvp),
                           static_cast<int64_t>(view.L.slots) * view.L.H);
  if (waves != nullptr) *waves = plan.waves;
  if (row_queue != nullptr) *row_queue = plan.row_queue ? 1 : 0;
  if (lds_bytes != nullptr) *lds_bytes = plan.lds_bytes;
  return 0;
}

int rosa_hip_measure_atomic_rate(void* buffer, size_t buffer_bytes, int row_floats, int columns,
                                 double* segments_per_second, void* stream) {
  if (buffer == nullptr || segments_per_second == nullptr) return fail(1, "NULL argument");
  if (row_floats < 16 || columns < 1 || columns > 16) return fail(1, "row_floats >= 16, 1 <= columns <= 16");
  const size_t rows = buffer_bytes / (sizeof(float) * static_cast<size_t>(row_floats));
  if (rows < 64 || rows > UINT32_MAX) return fail(1, "buffer holds too few or too many rows");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipEvent_t begin, end;
  if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess)
    return fail(5, "hipEventCreate failed");
  const int waves = kMaxResidentBlocks, tiles = 2000;
  // one short launch to warm up, then the timed one
  hipLaunchKernelGGL(atomic_rate_kernel, dim3(waves), dim3(kWave), 0, s, static_cast<float*>(buffer),
                     static_cast<uint32_t>(rows), static_cast<uint32_t>(row_floats), columns, 20);
  (void)hipEventRecord(begin, s);
  hipLaunchKernelGGL(atomic_rate_kernel, dim3(waves), dim3(kWave), 0, s, static_cast<float*>(buffer),
                     static_cast<uint32_t>(rows), static_cast<uint32_t>(row_floats), columns, tiles);
  (void)hipEventRecord(end, s);
  float ms = 0.0f;
  const bool ok = hipEventSynchronize(end) == hipSuccess &&
                  hipEventElapsedTime(&ms, begin, end) == hipSuccess && ms > 0.0f;
  (void)hipEventDestroy(begin);
  (void)hipEventDestroy(end);
  if (!ok) return fail(5, "timing the atomic kernel failed");
  // 16 row segments per tile
  *segments_per_second = static_cast<double>(waves) * tiles * 16.0 / (ms * 1e-3);
  return 0;
}

int rosa_hip_read_offset_error(const void* workspace, void* stream) {
  int32_t flag = 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (hipMemcpyAsync(&flag, workspace, sizeof(flag), hipMemcpyDeviceToHost, s) != hipSuccess)
    return -1;
  if (hipStreamSynchronize(s) != hipSuccess) return -1;
  return flag;
}

}  // extern "C"
