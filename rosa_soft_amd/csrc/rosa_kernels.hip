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

#include "rosa_vjp_bands.hpp"

#include <atomic>
#include <mutex>

// Scratch memory of rosa_hip_hard_forward_static: the forward's workspace (route of every
// row and the packed-sequence tables) for callers that cannot allocate.  Every device the
// library runs on holds its own copy until the process ends.  In host code the array's name
// is not a device address: the address of a device's copy comes from hipGetSymbolAddress.
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

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
// back, and the host waits for nothing, until rosa_hip_stage_times() or
// rosa_hip_stage_totals() is called.  Every stage keeps the events of its last
// kStageRing runs, so that a loop of calls can be timed without a wait per call.
enum Stage { kStageForward = 0, kStagePrepare, kStageRowMax, kStageRowStats, kStageGradients,
             kStageFinalize, kStageCount };
constexpr int kStageRing = 64;

struct StageTimer {
  bool enabled = false;
  bool created = false;
  hipEvent_t begin[kStageCount][kStageRing];
  hipEvent_t end[kStageCount][kStageRing];
  int64_t runs[kStageCount];   // since timing was enabled or the totals were last read
};

StageTimer g_timer;

void stage_begin(Stage stage, hipStream_t stream) {
  if (!g_timer.enabled) return;
  (void)hipEventRecord(g_timer.begin[stage][g_timer.runs[stage] % kStageRing], stream);
}

void stage_end(Stage stage, hipStream_t stream) {
  if (!g_timer.enabled) return;
  (void)hipEventRecord(g_timer.end[stage][g_timer.runs[stage] % kStageRing], stream);
  g_timer.runs[stage] += 1;
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

// Symbols of whole 16-byte pieces (D * element size a multiple of 16): a thread reads its
// symbol in 16-byte loads, and a block of kPackTokens tokens x H heads turns its words
// through LDS, so that they leave head-major in runs of kPackTokens consecutive tokens (the
// kernel above writes every word to a line of its own).  Dynamic LDS: two tiles of
// [H][kPackTokens + 1] words.
constexpr int kPackTokens = 16;
constexpr int kPackHeadsMax = 256;

template <int DTYPE>
__global__ __launch_bounds__(256) void pack_symbols_tile_kernel(
    const void* __restrict__ query, const void* __restrict__ key,
    int32_t* __restrict__ packed_query, int32_t* __restrict__ packed_key, int64_t tokens, int D,
    int H, int T, int N, int varlen) {
  extern __shared__ uint32_t pack_tile[];
  constexpr int kPiece = DTYPE == ROSA_DTYPE_F32 ? 4 : 8;  // elements in 16 bytes
  constexpr int kPitch = kPackTokens + 1;
  uint32_t* q_tile = pack_tile;
  uint32_t* k_tile = pack_tile + H * kPitch;
  const int64_t token0 = static_cast<int64_t>(blockIdx.x) * kPackTokens;
  const int here = static_cast<int>(min<int64_t>(kPackTokens, tokens - token0));
  const int rows = here * H;
  const int pieces = D / kPiece;
  const uint4* q_pieces = reinterpret_cast<const uint4*>(query) + token0 * H * pieces;
  const uint4* k_pieces = reinterpret_cast<const uint4*>(key) + token0 * H * pieces;
  for (int r = threadIdx.x; r < rows; r += blockDim.x) {
    uint32_t q_word = 0u, k_word = 0u;
    for (int piece = 0; piece < pieces; ++piece) {
      const uint4 q_in = q_pieces[static_cast<int64_t>(r) * pieces + piece];
      const uint4 k_in = k_pieces[static_cast<int64_t>(r) * pieces + piece];
#pragma unroll
      for (int e = 0; e < kPiece; ++e) {
        if (load_as_float<DTYPE>(&q_in, e) > 0.0f) q_word |= 1u << (piece * kPiece + e);
        if (load_as_float<DTYPE>(&k_in, e) > 0.0f) k_word |= 1u << (piece * kPiece + e);
      }
    }
    const int local = r / H;
    const int h = r - local * H;
    q_tile[h * kPitch + local] = q_word;
    k_tile[h * kPitch + local] = k_word;
  }
  __syncthreads();
  for (int index = threadIdx.x; index < H * kPackTokens; index += blockDim.x) {
    const int h = index / kPackTokens;
    const int local = index - h * kPackTokens;
    if (local >= here) continue;
    const int64_t token = token0 + local;
    int64_t dst;
    if (varlen) {
      dst = static_cast<int64_t>(h) * N + token;
    } else {
      const int64_t b = token / T;
      dst = (b * H + h) * T + (token - b * T);
    }
    packed_query[dst] = static_cast<int32_t>(q_tile[h * kPitch + local]);
    packed_key[dst] = static_cast<int32_t>(k_tile[h * kPitch + local]);
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

// `left_over` (or NULL): one byte per block of the grid; the kernel then routes only the
// row blocks whose byte is set, those that route_candidates_kernel has left to it.
template <bool VARLEN, bool WIDE>
__global__ __launch_bounds__(kWave) void hard_route_kernel(
    Layout L, const uint32_t* __restrict__ packed_query,
    const uint32_t* __restrict__ packed_key, int32_t* __restrict__ routes,
    int32_t* __restrict__ lengths, int32_t* __restrict__ source_token, int shift,
    const uint8_t* __restrict__ left_over) {
  if (left_over != nullptr && left_over[blockIdx.x] == 0) return;
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

// ---------------------------------------------------------------------------
// hard forward from an index of the keys
// ---------------------------------------------------------------------------
//
// A route a of row t has a run of at least one iff k[a - 1] == q[t], and its run is then the
// number of equal symbols walking back from there.  With symbols of many bits few routes of
// a row qualify (T / 2^bits of them on random symbols), so instead of stepping over every
// route a row can visit just those: index_keys_kernel sorts the key positions of every
// (sequence, head) into buckets by symbol (counting sort in LDS; an entry carries the route,
// its key symbol and the key symbol before it), and route_candidates_kernel lets every row
// walk its own bucket.  The winner is the same "longest first, latest on ties" maximum, so
// the routes are those of hard_route_kernel bit for bit.  Inputs this does not suit are
// handed back to the scan: a (sequence, head) whose largest bucket is far above the mean
// (few distinct symbols), and a row block whose walk exceeds its budget of iterations (long
// matches everywhere, as on periodic inputs); hard_route_kernel then runs for those blocks
// only.
constexpr int kIndexThreads = 1024;
constexpr int kIndexBucketsMax = 4096;

__device__ __forceinline__ uint32_t key_bucket(uint32_t symbol, int log_buckets, int hashed) {
  return hashed ? (symbol * 0x9e3779b1u) >> (32 - log_buckets) : symbol & ((1u << log_buckets) - 1u);
}

struct KeyIndex {
  int32_t* bucket_begin;  // [units][buckets + 1]
  uint4* entries;         // [symbol rows]: (route, key symbol, key symbol before it, 0), by bucket
  uint8_t* unit_scan;     // [units]: 1 = this (sequence, head) is left to the scan
  uint8_t* left_over;     // [blocks of the route grid]: 1 = this row block is left to the scan
  int log_buckets;
  int hashed;             // symbols of more bits than log_buckets: buckets by a multiplicative hash
  // what a row block may spend before it is handed back: budget_base + rows above it / 8
  // bucket entries per lane, and a quarter of that in steps of walking back along runs (two
  // dependent loads each; on random symbols a row block walks a handful of steps in all)
  int budget_base;
};

template <bool VARLEN>
__global__ __launch_bounds__(kIndexThreads) void index_keys_kernel(
    Layout L, const uint32_t* __restrict__ packed_key, KeyIndex index) {
  __shared__ int cursor[kIndexBucketsMax];
  __shared__ int partial[kIndexThreads];
  __shared__ int largest;
  const int unit = blockIdx.x;
  const int head = unit % L.H;
  const int seq = unit / L.H;
  int len;
  int64_t word_base;
  if constexpr (VARLEN) {
    len = L.seq_len[seq];
    word_base = static_cast<int64_t>(head) * L.N + L.seq_start[seq];
  } else {
    len = L.T;
    word_base = (static_cast<int64_t>(seq) * L.H + head) * L.T;
  }
  const int buckets = 1 << index.log_buckets;
  const int count = max(len - 1, 0);  // key positions 0 .. len - 2 carry routes 1 .. len - 1
  const uint32_t* k = packed_key + word_base;
  const int thread = threadIdx.x;
  for (int b = thread; b < buckets; b += kIndexThreads) cursor[b] = 0;
  if (thread == 0) largest = 0;
  __syncthreads();
  for (int p = thread; p < count; p += kIndexThreads)
    atomicAdd(&cursor[key_bucket(k[p], index.log_buckets, index.hashed)], 1);
  __syncthreads();
  // exclusive prefix sums: a thread owns `per` neighbouring buckets
  const int per = max(buckets / kIndexThreads, 1);
  const int first = thread * per;
  int mine = 0, biggest = 0;
  if (first < buckets) {
    for (int b = first; b < first + per; ++b) {
      mine += cursor[b];
      biggest = max(biggest, cursor[b]);
    }
  }
  partial[thread] = mine;
  atomicMax(&largest, biggest);
  __syncthreads();
  for (int step = 1; step < kIndexThreads; step <<= 1) {
    const int below = thread >= step ? partial[thread - step] : 0;
    __syncthreads();
    partial[thread] += below;
    __syncthreads();
  }
  int32_t* begin = index.bucket_begin + static_cast<int64_t>(unit) * (buckets + 1);
  if (first < buckets) {
    int running = partial[thread] - mine;
    for (int b = first; b < first + per; ++b) {
      const int size = cursor[b];
      cursor[b] = running;
      begin[b] = running;
      running += size;
    }
  }
  if (thread == 0) {
    begin[buckets] = count;
    // a bucket far above the mean: few distinct symbols, the scan is the better walk
    index.unit_scan[unit] = largest > max(64, count / 16) ? 1 : 0;
  }
  __syncthreads();
  // The positions go out in passes of kIndexThreads with a barrier between the passes: inside
  // a bucket the entries of an earlier pass then lie before those of a later one, and a row
  // can stop at the first entry of a pass that begins beyond it.
  uint4* entries = index.entries + word_base;
  for (int p0 = 0; p0 < count; p0 += kIndexThreads) {
    const int p = p0 + thread;
    if (p < count) {
      const uint32_t symbol = k[p];
      const int slot = atomicAdd(&cursor[key_bucket(symbol, index.log_buckets, index.hashed)], 1);
      entries[slot] = make_uint4(static_cast<uint32_t>(p + 1), symbol, p >= 1 ? k[p - 1] : 0u, 0u);
    }
    __syncthreads();
  }
}

template <bool VARLEN>
__global__ __launch_bounds__(kWave) void route_candidates_kernel(
    Layout L, const uint32_t* __restrict__ packed_query,
    const uint32_t* __restrict__ packed_key, int32_t* __restrict__ routes,
    int32_t* __restrict__ lengths, int32_t* __restrict__ source_token, KeyIndex index) {
  const Unit u = decode_unit<VARLEN>(L, blockIdx.x);
  const int lane = threadIdx.x;
  if (!u.valid) {
    if (lane == 0) index.left_over[blockIdx.x] = 0;
    return;
  }
  const int blocks = (u.len + 63) >> 6;
  if (u.block >= blocks) {
    if (lane == 0) index.left_over[blockIdx.x] = 0;
    return;
  }
  const int unit = u.seq * L.H + u.head;
  if (index.unit_scan[unit] != 0) {
    if (lane == 0) index.left_over[blockIdx.x] = 1;
    return;
  }
  const int row_block = blocks - 1 - u.block;  // as in hard_route_kernel
  const int t0 = row_block * kWave;
  const uint32_t* q = packed_query + u.word_base;
  const uint32_t* k = packed_key + u.word_base;
  const int t = t0 + lane;
  const bool row_ok = t < u.len;
  const uint32_t q_symbol = row_ok ? q[t] : 0u;
  const uint32_t q_before = (row_ok && t >= 1) ? q[t - 1] : 0u;
  const int buckets = 1 << index.log_buckets;
  const int32_t* begin = index.bucket_begin + static_cast<int64_t>(unit) * (buckets + 1);
  const uint32_t bucket = key_bucket(q_symbol, index.log_buckets, index.hashed);
  int next = row_ok ? begin[bucket] : 0;
  const int end = row_ok ? begin[bucket + 1] : 0;
  const uint4* entries = index.entries + u.word_base;
  const int budget = index.budget_base + t0 / 8;
  const int walk_budget = budget / 4;
  int spent = 0, walked = 0;  // wave-uniform
  uint64_t best = 0;  // (run << 32) | route
  uint4 ahead = next < end ? entries[next] : make_uint4(0u, 0u, 0u, 0u);
  while (__builtin_amdgcn_ballot_w64(next < end) != 0ull) {
    const bool have = next < end;
    const uint4 entry = ahead;
    ++next;
    if (next < end) ahead = entries[next];
    const int a = static_cast<int>(entry.x);
    // an entry of a pass of the index that begins beyond this row: so do all that follow
    if (have && ((a - 1) & ~(kIndexThreads - 1)) >= t) next = end;
    const bool candidate = have && a <= t && entry.y == q_symbol;
    const int limit = min(L.W, a);
    int run = candidate ? 1 : 0;
    bool walking = candidate && limit >= 2 && entry.z == q_before;
    if (walking) run = 2;
    walking = walking && run < limit;
    while (walked <= walk_budget && __builtin_amdgcn_ballot_w64(walking) != 0ull) {
      ++walked;
      if (walking) {
        if (q[t - run] == k[a - 1 - run]) {
          ++run;
          walking = run < limit;
        } else {
          walking = false;
        }
      }
    }
    const uint64_t found = (static_cast<uint64_t>(run) << 32) | static_cast<uint32_t>(a);
    if (candidate) best = max(best, found);
    if (++spent > budget || walked > walk_budget) {
      if (lane == 0) index.left_over[blockIdx.x] = 1;
      return;
    }
  }
  if (lane == 0) index.left_over[blockIdx.x] = 0;
  if (!row_ok) return;
  const int run = static_cast<int>(best >> 32);
  const int route = run > 0 ? static_cast<int>(best & 0xffffffffu) : 0;
  if (routes != nullptr) routes[u.word_base + t] = route;
  if (lengths != nullptr) lengths[u.word_base + t] = run;
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

// The same with 16 bytes of a row per thread, for value widths of whole 16-byte pieces.
template <int DTYPE>
__global__ __launch_bounds__(256) void gather_value_pieces_kernel(
    const int32_t* __restrict__ source_token, const void* __restrict__ value,
    void* __restrict__ output, int64_t pieces, int pieces_per_row, int H, int Hv, int Dv, int T,
    int N, int varlen, const int32_t* __restrict__ offset_error) {
  constexpr int kPiece = DTYPE == ROSA_DTYPE_F32 ? 4 : 8;  // elements in 16 bytes
  const int64_t piece = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (piece >= pieces) return;
  uint4 out = make_uint4(0u, 0u, 0u, 0u);
  if (offset_error != nullptr && *offset_error != 0) {
#pragma unroll
    for (int e = 0; e < kPiece; ++e) store_nan<DTYPE>(&out, e);
  } else {
    const int64_t row = piece / pieces_per_row;
    const int part = static_cast<int>(piece - row * pieces_per_row);
    const int64_t token = row / H;
    const int h = static_cast<int>(row - token * H);
    int64_t word;
    if (varlen) {
      word = static_cast<int64_t>(h) * N + token;
    } else {
      const int64_t b = token / T;
      word = (b * H + h) * T + (token - b * T);
    }
    const int source = source_token[word];
    if (source >= 0) {
      const int hv = h / (H / Hv);
      const uint4 in = reinterpret_cast<const uint4*>(value)[
          ((static_cast<int64_t>(source) * Hv + hv) * Dv) / kPiece + part];
#pragma unroll
      for (int e = 0; e < kPiece; ++e)
        store_sign<DTYPE>(&out, e, load_as_float<DTYPE>(&in, e) > 0.0f ? 1 : -1);
    }
  }
  reinterpret_cast<uint4*>(output)[piece] = out;
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

// SIMDs of the current device (the persistent gradient kernel keeps as many waves resident
// on each as it is compiled for): four per compute unit, the count read from the device's
// properties once per process (the devices of one node are alike).  Without a device (size
// queries on a host that has none) it is that of an MI355X, 256 compute units.
int device_simds() {
  static const int simds = [] {
    int device = 0;
    hipDeviceProp_t properties;
    if (hipGetDevice(&device) != hipSuccess ||
        hipGetDeviceProperties(&properties, device) != hipSuccess ||
        properties.multiProcessorCount <= 0) {
      (void)hipGetLastError();  // not an error of the call that asked
      return 4 * 256;
    }
    return 4 * properties.multiProcessorCount;
  }();
  return simds;
}

// blocks of the gradient kernel that are resident at two waves per SIMD
int max_resident_blocks() { return 2 * device_simds(); }
int resident_gradient_waves(int value_tiles, int symbol_tiles) {
  return device_simds() * (gradient_waves(value_tiles, symbol_tiles) < 2
                     ? 2 : gradient_waves(value_tiles, symbol_tiles));
}

// Waves per block of the gradient kernel (rosa_hip_set_gradient_block_waves overrides).
// Two waves halve the column atomics, which bound the wide tiles; the narrow tile is bound
// by its arithmetic, and with few bands per resident wave the kernel's time is that of
// its longest band, which a block of two waves walks more slowly than a single wave.
// (the knobs are atomics so that a setter racing with a size query or a launch is not
// undefined; the two may still see different values, see the header)
std::atomic<int> g_gradient_block_waves{0};  // 0: by shape

// Rows of a piece of a band in the gradient kernel (rosa_hip_set_gradient_piece_rows
// overrides): 0 by shape, -1 never, otherwise that many rows.
std::atomic<int> g_gradient_piece_rows{0};

// How the bands of the gradient kernel are cut into pieces (vjp_gradients_kernel): only with
// single-wave blocks and when there are fewer than two bands per resident wave, so that the
// longest band no longer sets the kernel's time.  A piece is at least four windows long (the
// W - 1 rows below it are walked a second time) and a whole number of staged segments.
struct PiecePlan {
  int piece_rows;   // 0: whole bands
  int max_pieces;   // work items per band
};

PiecePlan plan_band_pieces(int64_t units, int longest, int W, int64_t resident_waves, int segment) {
  PiecePlan plan{0, 1};
  const auto whole_segments = [&](int64_t rows) {
    return static_cast<int>((std::max<int64_t>(rows, 2 * segment) + segment - 1) / segment * segment);
  };
  int rows = 0;
  const int forced_rows = g_gradient_piece_rows.load(std::memory_order_relaxed);
  if (forced_rows > 0) {
    rows = whole_segments(forced_rows);
  } else if (forced_rows == 0 && g_gradient_block_waves.load(std::memory_order_relaxed) != 2 &&
             units > 0 &&
             units < 2 * resident_waves) {
    const int64_t pieces_wanted = (2 * resident_waves + units - 1) / units;
    rows = std::max(whole_segments(4 * static_cast<int64_t>(W)),
                    whole_segments((longest - 1 + pieces_wanted - 1) / pieces_wanted));
  }
  if (rows <= 0 || longest - 1 <= rows) return plan;
  const int64_t pieces = (static_cast<int64_t>(longest) - 1 + rows - 1) / rows;
  if (units * pieces > INT32_MAX) return plan;
  plan.piece_rows = rows;
  plan.max_pieces = static_cast<int>(pieces);
  return plan;
}


// How the gradient kernel is launched for a tile shape: waves per block, whether row tiles
// are queued between the bands of a block, and the LDS of a block.
struct GradientBlockPlan {
  int waves;
  bool row_queue;
  size_t wave_floats, tile_floats, lds_bytes;
};

int gradient_block_waves(int dvp, int symbol_tiles, int64_t units) {
  const int forced = g_gradient_block_waves.load(std::memory_order_relaxed);
  if (forced == 1 || forced == 2) return forced;
  return ((dvp >= 16 || symbol_tiles > 1) && units >= 2 * max_resident_blocks()) ? 2 : 1;
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
  // the index of the keys (route_candidates_kernel); log_buckets == 0: no room for it
  int log_buckets, hashed;
  size_t bucket_begin, entries, unit_scan, left_over;
};

// Shapes the index of the keys is used for unless the caller says otherwise: symbols of six
// bits or more (below that most routes of a row match and the scan is the better walk) and
// sequences long enough for the two extra launches to pay.  The workspace has room for it
// at every shape, so that the choice can be made per launch.
constexpr int kIndexSymbolBitsMin = 6;
constexpr int kIndexLongestMin = 512;
constexpr int64_t kIndexRowsMax = int64_t(1) << 26;

ForwardWorkspace carve_forward(const ProblemView& v, bool with_index = true) {
  ForwardWorkspace w;
  size_t cursor = 0;
  w.header = cursor; cursor += align_up(256);
  const size_t s = static_cast<size_t>(v.L.varlen ? v.L.S : 0);
  w.seq_start = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.seq_len = cursor; cursor += align_up(sizeof(int32_t) * s);
  w.block_prefix = cursor; cursor += align_up(sizeof(int32_t) * (s + 1));
  w.source_token = cursor; cursor += align_up(sizeof(int32_t) * static_cast<size_t>(v.symbol_rows));
  w.log_buckets = 0; w.hashed = 0;
  w.bucket_begin = w.entries = w.unit_scan = w.left_over = 0;
  const int longest = v.L.varlen ? v.L.N : v.L.T;
  // (beyond 64 M rows, 1.5 GiB of index, the forward keeps to the scan and its 4 bytes per row)
  if (with_index && v.symbol_rows <= kIndexRowsMax) {
    // about four keys per bucket on the longest sequence, at most one bucket per symbol
    int log_buckets = 6;
    while (log_buckets < 12 && (4 << log_buckets) < longest) ++log_buckets;
    const size_t units = static_cast<size_t>(v.L.varlen ? v.L.S : v.L.B) * v.L.H;
    // (many short packed sequences: the bucket tables stay below four bytes per token and head)
    while (log_buckets > 1 && (units << log_buckets) > static_cast<size_t>(v.symbol_rows)) --log_buckets;
    w.hashed = v.L.D > log_buckets ? 1 : 0;
    w.log_buckets = std::min(log_buckets, v.L.D);
    const size_t blocks = static_cast<size_t>(v.L.slots) * v.L.H;
    w.bucket_begin = cursor;
    cursor += align_up(sizeof(int32_t) * units * ((size_t(1) << w.log_buckets) + 1));
    w.entries = cursor; cursor += align_up(sizeof(uint4) * static_cast<size_t>(v.symbol_rows));
    w.unit_scan = cursor; cursor += align_up(units);
    w.left_over = cursor; cursor += align_up(blocks);
  }
  w.total = cursor;
  return w;
}

// rosa_hip_set_forward_index: 0 = the index at the shapes above, 1 = never, 2 = the index
// with no budget at all (every row block is handed back to the scan), 3 = the index at
// every shape (2 and 3 are for tests)
std::atomic<int> g_forward_index_mode{0};

constexpr int kValueSlice = 64;  // value dimensions one backward pass covers
constexpr int kNarrowRow = 8;    // gradient rows up to this many floats are accumulated head-major

// bytes of chunk records the backward workspace may hold unless the caller sets a limit:
// at most 4 GiB, and in a packed layout, whose sequence lengths the host does not know, at
// most 1.5 KiB per token and head (what sequences of about 6 000 tokens need with dropout;
// longer ones make the device fall back to rebuilding the evidence in the gradient pass)
constexpr size_t kDefaultRecordBudget = size_t(1) << 32;
constexpr size_t kPackedRecordBytesPerRow = 1536;
constexpr size_t kNoRecordBudget = static_cast<size_t>(-1);
std::atomic<size_t> g_record_budget_bytes{kNoRecordBudget};  // set by rosa_hip_set_record_budget

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
    size_t budget_bytes = g_record_budget_bytes.load(std::memory_order_relaxed);
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
  // (the ring holds a float and a bfloat16 per row and lane)
  w.block_scratch_floats = static_cast<int64_t>(w.ring_rows) * (kWave + kWave / 2) +
                           2 * kCheckpointChunksMax * kWave +
                           static_cast<int64_t>(max_segments > 0 ? max_groups + w.segment_group : 0) *
                               2 * kWave;
  const int64_t units = static_cast<int64_t>(v.L.slots) * v.L.H;
  // resident waves of the gradient kernel (an even number: its blocks hold one or two waves)
  const int64_t resident_cap = resident_gradient_waves((dvp + 15) / 16, v.L.D > 16 ? 2 : 1);
  const PiecePlan pieces = plan_band_pieces(units, longest, v.L.W, resident_cap, segment_rows);
  w.resident_blocks = static_cast<int>(
      std::min<int64_t>((units * pieces.max_pieces + 1) & ~int64_t(1), resident_cap));
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
                bool words_given = false, bool allow_index = true) {
  Layout L = view.L;
  const ForwardWorkspace w = carve_forward(view, allow_index);
  stage_begin(kStageForward, stream);
  launch_prepare_sequences(p, L, workspace, w.seq_start, w.seq_len, w.block_prefix, w.header,
                           stream);
  const int64_t elements = view.symbol_rows * L.D;
  constexpr int kPackPiece = DTYPE == ROSA_DTYPE_F32 ? 4 : 8;  // elements in 16 bytes
  const bool whole_symbol_pieces =
      L.D % kPackPiece == 0 && L.H <= kPackHeadsMax &&
      ((reinterpret_cast<uintptr_t>(query) | reinterpret_cast<uintptr_t>(key)) & 15u) == 0;
  if (words_given) {
    // a producer (the projection in front of the operator) has written the symbol words
  } else if (whole_symbol_pieces) {
    const size_t tile_bytes = sizeof(uint32_t) * 2 * static_cast<size_t>(L.H) * (kPackTokens + 1);
    hipLaunchKernelGGL(pack_symbols_tile_kernel<DTYPE>,
                       dim3(blocks_for(view.tokens, kPackTokens)), dim3(256), tile_bytes, stream,
                       query, key, packed_query, packed_key, view.tokens, L.D, L.H, L.T, L.N,
                       L.varlen);
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
  const int index_mode = g_forward_index_mode.load(std::memory_order_relaxed);
  const uint8_t* left_over = nullptr;
  // (a packed batch is judged by its mean sequence length: the host does not know the
  // lengths, and a block per (sequence, head) costs more than it saves on short sequences)
  const int typical = L.varlen ? L.N / std::max(L.S, 1) : L.T;
  const bool index_suits = L.D >= kIndexSymbolBitsMin && typical >= kIndexLongestMin;
  if (w.log_buckets > 0 && (index_mode >= 2 || (index_mode == 0 && index_suits))) {
    KeyIndex index;
    index.bucket_begin = at<int32_t>(workspace, w.bucket_begin);
    index.entries = at<uint4>(workspace, w.entries);
    index.unit_scan = at<uint8_t>(workspace, w.unit_scan);
    index.left_over = at<uint8_t>(workspace, w.left_over);
    index.log_buckets = w.log_buckets;
    index.hashed = w.hashed;
    index.budget_base = index_mode == 2 ? -(1 << 30) : 64;
    const unsigned sequences = static_cast<unsigned>(L.varlen ? L.S : L.B) * static_cast<unsigned>(L.H);
    if (L.varlen) {
      hipLaunchKernelGGL(index_keys_kernel<true>, dim3(sequences), dim3(kIndexThreads), 0, stream,
                         L, pk, index);
      hipLaunchKernelGGL(route_candidates_kernel<true>, dim3(units), dim3(kWave), 0, stream, L, pq,
                         pk, routes, lengths, source_token, index);
    } else {
      hipLaunchKernelGGL(index_keys_kernel<false>, dim3(sequences), dim3(kIndexThreads), 0, stream,
                         L, pk, index);
      hipLaunchKernelGGL(route_candidates_kernel<false>, dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, index);
    }
    left_over = index.left_over;
  }
  if (L.varlen) {
    if (wide) {
      hipLaunchKernelGGL((hard_route_kernel<true, true>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift, left_over);
    } else {
      hipLaunchKernelGGL((hard_route_kernel<true, false>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift, left_over);
    }
  } else {
    if (wide) {
      hipLaunchKernelGGL((hard_route_kernel<false, true>), dim3(units), dim3(kWave), 0, stream, L,
                         pq, pk, routes, lengths, source_token, shift, left_over);
    } else {
      hipLaunchKernelGGL((hard_route_kernel<false, false>), dim3(units), dim3(kWave), 0, stream,
                         L, pq, pk, routes, lengths, source_token, shift, left_over);
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
    constexpr int kPiece = DTYPE == ROSA_DTYPE_F32 ? 4 : 8;  // elements in 16 bytes
    const bool whole_pieces =
        L.Dv % kPiece == 0 &&
        ((reinterpret_cast<uintptr_t>(value) | reinterpret_cast<uintptr_t>(output)) & 15u) == 0;
    if (whole_pieces) {
      const int64_t pieces = out_elements / kPiece;
      hipLaunchKernelGGL(gather_value_pieces_kernel<DTYPE>, dim3(blocks_for(pieces, 256)),
                         dim3(256), 0, stream, source_token, value, output, pieces,
                         L.Dv / kPiece, L.H, L.Hv, L.Dv, L.T, L.N, L.varlen, offset_error);
    } else {
      hipLaunchKernelGGL(gather_values_kernel<DTYPE>, dim3(blocks_for(out_elements, 256)),
                         dim3(256), 0, stream, source_token, value, output, out_elements, L.H,
                         L.Hv, L.Dv, L.T, L.N, L.varlen, offset_error);
    }
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

// The band kernels are compiled in translation units of their own, one per tile family
// (sign words per value column, padded value width, symbol tiles); each exports its table
// of kernel addresses (see vjp_kernel_slot in rosa_vjp_bands.hpp).
extern "C" {
const void* const* rosa_vjp_kernels_1_8_1(void);
const void* const* rosa_vjp_kernels_1_8_2(void);
const void* const* rosa_vjp_kernels_1_16_1(void);
const void* const* rosa_vjp_kernels_1_16_2(void);
const void* const* rosa_vjp_kernels_1_32_1(void);
const void* const* rosa_vjp_kernels_1_32_2(void);
const void* const* rosa_vjp_kernels_2_64_1(void);
const void* const* rosa_vjp_kernels_2_64_2(void);
}

const void* const* vjp_kernel_table(int dvp, int symbol_tiles) {
  const bool wide = symbol_tiles > 1;
  switch (dvp) {
    case 8: return wide ? rosa_vjp_kernels_1_8_2() : rosa_vjp_kernels_1_8_1();
    case 16: return wide ? rosa_vjp_kernels_1_16_2() : rosa_vjp_kernels_1_16_1();
    case 32: return wide ? rosa_vjp_kernels_1_32_2() : rosa_vjp_kernels_1_32_1();
    case 64: return wide ? rosa_vjp_kernels_2_64_2() : rosa_vjp_kernels_2_64_1();
    default: return nullptr;
  }
}

int launch_band_kernel(const void* kernel, unsigned blocks, unsigned threads, size_t lds_bytes,
                       hipStream_t stream, VjpParams& params) {
  if (kernel == nullptr) return fail(1, "no kernel for this tile shape");
  void* arguments[] = {&params};
  const hipError_t status =
      hipLaunchKernel(kernel, dim3(blocks), dim3(threads), arguments, lds_bytes, stream);
  return status == hipSuccess ? 0 : fail_hip(status, "launch of a band kernel");
}

// nvw: sign words per value column, dvp: padded value width, symbol_tiles: 1 or 2
int launch_vjp_passes(int nvw, int dvp, int symbol_tiles, bool dropout, const VjpParams& P,
                      const VjpWorkspace& w, bool analytic, hipStream_t stream) {
  const void* const* kernels = vjp_kernel_table(dvp, symbol_tiles);
  // the row kernels do not depend on the symbol tiles: they live in the one-tile family
  const void* const* row_kernels = vjp_kernel_table(dvp, 1);
  if (kernels == nullptr || row_kernels == nullptr) return fail(1, "no kernels for this tile shape");
  const int varlen = P.L.varlen != 0;
  const unsigned units = static_cast<unsigned>(P.total_units);
  VjpParams Q = P;
  int status = 0;
  if (!analytic) {
    stage_begin(kStageRowMax, stream);
    status = launch_band_kernel(row_kernels[vjp_kernel_slot_row_max(varlen)], units, kWave, 0,
                                stream, Q);
    stage_end(kStageRowMax, stream);
    if (status != 0) return status;
  }
  stage_begin(kStageRowStats, stream);
  status = launch_band_kernel(row_kernels[vjp_kernel_slot_row_stats(varlen, dropout)], units,
                              kWave, row_stats_dynamic_lds(P.grad_pitch), stream, Q);
  if (status != 0) return status;
  {
    const int64_t rows = static_cast<int64_t>(P.L.N) * P.L.H;
    hipLaunchKernelGGL(finalize_row_records_kernel, dim3(blocks_for(rows, 256)), dim3(256), 0,
                       stream, P.stats, rows, P.null_logit);
  }
  stage_end(kStageRowStats, stream);
  const int segment = gradient_segment(dvp);
  const GradientBlockPlan plan = plan_gradient_blocks(dvp, P.L.D, nvw, P.grad_pitch, P.total_units);
  Q.wave_lds_floats = static_cast<int>(plan.wave_floats);
  Q.exchange_tile_floats = static_cast<int>(plan.tile_floats);
  Q.row_queue = plan.row_queue ? 1 : 0;
  Q.piece_rows = 0;
  Q.max_pieces = 1;
  if (plan.waves == 1) {
    const PiecePlan pieces = plan_band_pieces(
        P.total_units, P.L.varlen ? P.L.N : P.L.T, P.L.W,
        resident_gradient_waves((dvp + 15) / 16, symbol_tiles), segment);
    Q.piece_rows = pieces.piece_rows;
    Q.max_pieces = pieces.max_pieces;
    Q.total_units = P.total_units * pieces.max_pieces;
  }
  const unsigned blocks = static_cast<unsigned>(std::max(1, w.resident_blocks / plan.waves));
  const int form = plan.waves == 2 ? kGradientFormTwoWaves
                                   : Q.piece_rows > 0 ? kGradientFormPieces : kGradientFormOneWave;
  stage_begin(kStageGradients, stream);
  // both forms of the kernel (see its TERMS): the one that does not apply returns at once
  for (int terms = 2; terms <= 3 && status == 0; ++terms) {
    status = launch_band_kernel(kernels[vjp_kernel_slot_gradients(varlen, dropout, form, terms)],
                                blocks, kWave * plan.waves, plan.lds_bytes, stream, Q);
  }
  stage_end(kStageGradients, stream);
  return status;
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
      status = launch_vjp_passes(1, dvp, P.L.D > 16 ? 2 : 1, dropout, P, w, analytic, stream);
    } else {
      status = launch_vjp_passes(2, 64, P.L.D > 16 ? 2 : 1, dropout, P, w, analytic, stream);
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
  int32_t* history_lengths_out;  // [S] or NULL: where the advanced lengths go instead
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
  // the index of the keys of every run, rebuilt by an update that uses it (NULL: none)
  int32_t* bucket_begin;         // [runs][2^qk_bits + 1]
  uint2* bucket_routes;          // [runs][index_stride]: (route, key symbol before it), by bucket
  uint8_t* run_scan;             // [runs]: 1 = the run is left to the scan
  uint8_t* left_over;            // [blocks of the routing grid]: 1 = left to the scan
  int index_stride;
  int log_buckets;
  int budget_base;
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
  // (behind router_candidates_kernel: only the row blocks that kernel has left over)
  if (U.left_over != nullptr && U.left_over[blockIdx.x] == 0) return;
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

// The index of the keys for the router (see index_keys_kernel): byte symbols, one bucket per
// symbol, the whole history of a run indexed anew by every update that routes a long chunk.
// An entry is the route and the key symbol before it; the key symbol itself is the bucket's.
__global__ __launch_bounds__(kIndexThreads) void router_index_kernel(RouterUpdate U) {
  __shared__ int cursor[256];
  __shared__ int partial[256];
  __shared__ int largest;
  const int run = blockIdx.x;
  const int slot = run / U.H;
  const int new_length = U.history_lengths[slot] +
                         (router_chunk_begin(U, slot + 1) - router_chunk_begin(U, slot));
  const int count = max(new_length - 1, 0);
  const int buckets = 1 << U.log_buckets;
  const uint8_t* k = U.key_history + static_cast<int64_t>(run) * U.capacity;
  const int thread = threadIdx.x;
  if (count > U.index_stride) {
    // the caller's longest_total was too small for this run: no room for its routes, the scan
    // takes it
    if (thread == 0) U.run_scan[run] = 1;
    return;
  }
  if (thread < 256) cursor[thread] = 0;
  if (thread == 0) largest = 0;
  __syncthreads();
  for (int p = thread; p < count; p += kIndexThreads) atomicAdd(&cursor[k[p]], 1);
  __syncthreads();
  const int mine = thread < buckets ? cursor[thread] : 0;
  if (thread < 256) partial[thread] = mine;
  if (thread < buckets) atomicMax(&largest, mine);
  __syncthreads();
  for (int step = 1; step < 256; step <<= 1) {
    const int below = (thread < 256 && thread >= step) ? partial[thread - step] : 0;
    __syncthreads();
    if (thread < 256) partial[thread] += below;
    __syncthreads();
  }
  int32_t* begin = U.bucket_begin + static_cast<int64_t>(run) * (buckets + 1);
  if (thread < buckets) {
    cursor[thread] = partial[thread] - mine;
    begin[thread] = partial[thread] - mine;
  }
  if (thread == 0) {
    begin[buckets] = count;
    U.run_scan[run] = largest > max(64, count / 16) ? 1 : 0;
  }
  __syncthreads();
  uint2* routes = U.bucket_routes + static_cast<int64_t>(run) * U.index_stride;
  for (int p0 = 0; p0 < count; p0 += kIndexThreads) {  // ordered passes, as in index_keys_kernel
    const int p = p0 + thread;
    if (p < count) {
      // (route 1 has no key before it: a value no symbol takes)
      routes[atomicAdd(&cursor[k[p]], 1)] =
          make_uint2(static_cast<uint32_t>(p + 1), p >= 1 ? static_cast<uint32_t>(k[p - 1]) : 0x100u);
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kWave) void router_candidates_kernel(RouterUpdate U) {
  const int run = static_cast<int>(blockIdx.x / static_cast<unsigned>(U.blocks_per_run));
  const int row_block = static_cast<int>(blockIdx.x - static_cast<unsigned>(run) * U.blocks_per_run);
  const int slot = run / U.H;
  const int head = run - slot * U.H;
  const int lane = threadIdx.x;
  const int old_length = U.history_lengths[slot];
  const int chunk_begin = router_chunk_begin(U, slot);
  const int new_length = old_length + (router_chunk_begin(U, slot + 1) - chunk_begin);
  const int t0 = old_length + row_block * kWave;
  if (t0 >= new_length || U.run_scan[run] != 0) {
    if (lane == 0) U.left_over[blockIdx.x] = t0 < new_length ? 1 : 0;
    return;
  }
  const int64_t run_base = static_cast<int64_t>(run) * U.capacity;
  const uint8_t* q = U.query_history + run_base;
  const uint8_t* k = U.key_history + run_base;
  const int t = t0 + lane;
  const bool row_ok = t < new_length;
  const uint32_t q_symbol = row_ok ? q[t] : 0u;
  const uint32_t q_before = (row_ok && t >= 1) ? q[t - 1] : 0u;
  const int buckets = 1 << U.log_buckets;
  const int32_t* begin = U.bucket_begin + static_cast<int64_t>(run) * (buckets + 1);
  int next = row_ok ? begin[q_symbol] : 0;
  const int end = row_ok ? begin[q_symbol + 1] : 0;
  const uint2* routes = U.bucket_routes + static_cast<int64_t>(run) * U.index_stride;
  const int budget = U.budget_base + t0 / 8;
  const int walk_budget = budget / 4;
  int spent = 0, walked = 0;  // wave-uniform
  uint64_t best = 0;          // (run << 32) | route
  uint2 ahead = next < end ? routes[next] : make_uint2(0u, 0x100u);
  while (__builtin_amdgcn_ballot_w64(next < end) != 0ull) {
    const bool have = next < end;
    const int a = static_cast<int>(ahead.x);
    const uint32_t key_before = ahead.y;
    ++next;
    if (next < end) ahead = routes[next];
    if (have && ((a - 1) & ~(kIndexThreads - 1)) >= t) next = end;
    const bool candidate = have && a <= t;
    const int limit = min(U.W, a);
    int length = candidate ? 1 : 0;
    bool walking = candidate && limit >= 2 && key_before == q_before;
    if (walking) length = 2;
    walking = walking && length < limit;
    while (walked <= walk_budget && __builtin_amdgcn_ballot_w64(walking) != 0ull) {
      ++walked;
      if (walking) {
        if (q[t - length] == k[a - 1 - length]) {
          ++length;
          walking = length < limit;
        } else {
          walking = false;
        }
      }
    }
    const uint64_t found = (static_cast<uint64_t>(length) << 32) | static_cast<uint32_t>(a);
    if (candidate) best = max(best, found);
    if (++spent > budget || walked > walk_budget) {
      if (lane == 0) U.left_over[blockIdx.x] = 1;
      return;
    }
  }
  if (lane == 0) U.left_over[blockIdx.x] = 0;
  if (!row_ok) return;
  const int route = (best >> 32) > 0 ? static_cast<int>(best & 0xffffffffu) : 0;
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
  const int chunk = router_chunk_begin(U, slot + 1) - router_chunk_begin(U, slot);
  if (U.history_lengths_out != nullptr) {
    U.history_lengths_out[slot] = U.history_lengths[slot] + chunk;
  } else {
    U.history_lengths[slot] += chunk;
  }
}

// A decoding step as one launch: where the advanced lengths go to an array of their own, a
// wave can append its row, route it and leave the new length without waiting for any other
// wave (three launches otherwise: append, route, advance, each waiting for the one before).
// Symbols at positions from the old length on are the chunk's own and are read from the
// update's inputs, so that no wave depends on another's append.
__global__ __launch_bounds__(kWave) void router_decode_step_kernel(RouterUpdate U) {
  const int run = static_cast<int>(blockIdx.x / static_cast<unsigned>(U.blocks_per_run));
  const int row = static_cast<int>(blockIdx.x - static_cast<unsigned>(run) * U.blocks_per_run);
  const int slot = run / U.H;
  const int head = run - slot * U.H;
  const int lane = threadIdx.x;
  const int old_length = U.history_lengths[slot];
  const int chunk_begin = router_chunk_begin(U, slot);
  const int rows = router_chunk_begin(U, slot + 1) - chunk_begin;
  if (head == 0 && row == 0 && lane == 0) U.history_lengths_out[slot] = old_length + rows;
  if (row >= rows) return;
  const int t = old_length + row;
  const int64_t run_base = static_cast<int64_t>(run) * U.capacity;
  const uint8_t* q_history = U.query_history + run_base;
  const uint8_t* k_history = U.key_history + run_base;
  const uint8_t* q_new = U.query + static_cast<int64_t>(chunk_begin) * U.H + head;
  const uint8_t* k_new = U.key + static_cast<int64_t>(chunk_begin) * U.H + head;
  const auto q_at = [&](int position) -> uint32_t {
    return position < old_length
        ? q_history[position]
        : q_new[static_cast<int64_t>(position - old_length) * U.H] & U.qk_mask;
  };
  const auto k_at = [&](int position) -> uint32_t {
    return position < old_length
        ? k_history[position]
        : k_new[static_cast<int64_t>(position - old_length) * U.H] & U.qk_mask;
  };
  const int payload_head = head / (U.H / U.Hp);
  const int64_t payload_base = (static_cast<int64_t>(slot) * U.Hp + payload_head) * U.capacity;
  if (lane == 0) {  // this row's symbols join the histories
    U.query_history[run_base + t] = static_cast<uint8_t>(q_at(t));
    U.key_history[run_base + t] = static_cast<uint8_t>(k_at(t));
    if (head < U.Hp) {
      U.payload_history[(static_cast<int64_t>(slot) * U.Hp + head) * U.capacity + t] =
          U.payload[static_cast<int64_t>(chunk_begin + row) * U.Hp + head] & U.payload_mask;
    }
  }
  const uint32_t q_symbol = q_at(t);
  unsigned long long best = 0ull;
  constexpr int kAhead = 4;  // key symbols a lane has in flight
  for (int a0 = 1 + lane; a0 <= t; a0 += kAhead * kWave) {
    uint32_t keys[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int a = a0 + j * kWave;
      keys[j] = a <= t ? k_at(a - 1) : 0x100u;
    }
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      if (keys[j] != q_symbol) continue;
      const int a = a0 + j * kWave;
      const int limit = min(U.W, a);
      int length = 1;
      while (length < limit && q_at(t - length) == k_at(a - 1 - length)) ++length;
      best = max(best, (static_cast<unsigned long long>(length) << 32) | static_cast<uint32_t>(a));
    }
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    best = max(best, static_cast<unsigned long long>(__shfl_xor(best, offset, kWave)));
  }
  if (lane != 0) return;
  const int route = (best >> 32) > 0 ? static_cast<int>(best & 0xffffffffull) : 0;
  const int64_t token = chunk_begin + row;
  uint8_t symbol = 0;
  if (route > 0) {  // the payload that follows the matched key: position `route`
    symbol = route < old_length
        ? U.payload_history[payload_base + route]
        : U.payload[static_cast<int64_t>(chunk_begin + route - old_length) * U.Hp + payload_head] &
              U.payload_mask;
  }
  U.matched_key_end[token * U.H + head] = route > 0 ? route - 1 : -1;
  U.output[token * U.H + head] = symbol;
}

// ---------------------------------------------------------------------------
// the projection that follows the operator, fed with the bit form of its output
// ---------------------------------------------------------------------------
//
//   out[t, n] = residual[t, n] + sum_k y[t, k] * weight[n, k],   k = h * Dv + d,
//   y[t, k] = routed[t, h] ? (bit d of sign_words[t, h] ? +1 : -1) : 0
//
// i.e. `residual + output(routed.flatten(2))` of the reference's caller
// (examples/fit_soft_reference.py:374-417) without the ternary tensor in between: the
// operand of the matrix products that holds y is expanded from the bits in registers (the
// weights are the products' row operand, so that a lane ends up with four neighbouring
// output columns of one token).  `weight` is the
// [N][K] matrix of a linear layer (k contiguous), bfloat16; accumulation is float32.
// A block of four waves computes 256 rows x 64 columns, each wave 64 x 64 (sixteen
// 16 x 16 x 32 products per 32-wide k step).  Per staged step of 64 k (two products deep) a
// block stages the weight tile [64][64] and, per row, the sign and validity bits of the step
// in LDS; the loads of the next step are in flight while the products of this one run.
constexpr int kProjectRows = 256;
constexpr int kProjectColumns = 64;
constexpr int kProjectStep = 32;    // k of one matrix product, and what K must be a multiple of
// k staged per barrier (128 needs registers beyond three waves per SIMD, and is slower for it)
constexpr int kProjectStage = 64;
constexpr int kStageProducts = kProjectStage / kProjectStep;
constexpr int kProjectWeightPitch = kProjectStage + 8;  // bfloat16 elements per staged weight row

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

// Sign bits and validity bits of k = 32 step .. 32 step + 31 of one token.  HEADS: heads per
// step (4: value width 8, 2: width 16), or 0 where a head spans whole steps (a width that is
// a multiple of 32: step `step` is then word `step` of the token's words).
template <int HEADS>
__device__ __forceinline__ uint2 ternary_step_bits(const ProjectParams& P, int64_t token, int step) {
  uint32_t signs = 0u, valid = 0u;
  if (token < P.tokens) {
    if constexpr (HEADS == 0) {
      signs = P.sign_words[token * P.H * P.nvw + step];
      valid = P.routed[token * P.H + step / P.nvw] == 1 ? 0xffffffffu : 0u;
    } else if constexpr (HEADS == 2) {
      const int64_t first = token * P.H + 2 * step;
      const uint2 words = *reinterpret_cast<const uint2*>(P.sign_words + first);
      const uint32_t flags = *reinterpret_cast<const uint16_t*>(P.routed + first);
      signs = (words.x & 0xffffu) | (words.y << 16);
      valid = ((flags & 0xffu) == 1u ? 0xffffu : 0u) | ((flags >> 8) == 1u ? 0xffff0000u : 0u);
    } else {
      static_assert(HEADS == 4, "a step holds four, two or a part of one head");
      const int64_t first = token * P.H + 4 * step;
      const uint4 words = *reinterpret_cast<const uint4*>(P.sign_words + first);
      const uint32_t flags = *reinterpret_cast<const uint32_t*>(P.routed + first);
      signs = (words.x & 0xffu) | ((words.y & 0xffu) << 8) | ((words.z & 0xffu) << 16) | (words.w << 24);
      valid = ((flags & 0xffu) == 1u ? 0xffu : 0u) | (((flags >> 8) & 0xffu) == 1u ? 0xff00u : 0u) |
              (((flags >> 16) & 0xffu) == 1u ? 0xff0000u : 0u) | ((flags >> 24) == 1u ? 0xff000000u : 0u);
    }
  }
  return make_uint2(signs, valid);
}

template <int HEADS>
__global__ __launch_bounds__(256) void project_routed_bits_kernel(ProjectParams P) {
  __shared__ __attribute__((aligned(16))) uint16_t weight_tile[2][kProjectColumns * kProjectWeightPitch];
  // (signs, valid) of every product of the stage, per row
  __shared__ __attribute__((aligned(16))) uint2 row_bits[2][kProjectRows][kStageProducts];
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
  const int products = P.K / kProjectStep;           // 32-wide k steps in all
  const int stages = (products + kStageProducts - 1) / kStageProducts;
  // what a thread stages per stage: a quarter of one weight row's stage and one row's bits
  constexpr int kThreadElements = kProjectStage / 4;
  constexpr int kThreadChunks = kThreadElements / 8;   // of 16 bytes
  const int stage_n = thread >> 2;
  const int stage_k = (thread & 3) * kThreadElements;
  const uint16_t* weight_row = P.weight + static_cast<int64_t>(n0 + stage_n) * P.K + stage_k;
  uint4 weight_in[kThreadChunks];
  uint2 bits_in[kStageProducts];
  const auto fetch_stage = [&](int stage) {
    // (K is a multiple of 32: the last stage may hold fewer products than the others)
#pragma unroll
    for (int chunk = 0; chunk < kThreadChunks; ++chunk) {
      const int k = stage * kProjectStage + stage_k + 8 * chunk;
      weight_in[chunk] = k + 8 <= P.K
                             ? *reinterpret_cast<const uint4*>(weight_row + stage * kProjectStage + 8 * chunk)
                             : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int h = 0; h < kStageProducts; ++h) {
      const int step = stage * kStageProducts + h;
      bits_in[h] = step < products ? ternary_step_bits<HEADS>(P, row0 + thread, step) : make_uint2(0u, 0u);
    }
  };
  fetch_stage(0);
  for (int stage = 0; stage < stages; ++stage) {
    const int buffer = stage & 1;
    uint16_t* staged = &weight_tile[buffer][stage_n * kProjectWeightPitch + stage_k];
#pragma unroll
    for (int chunk = 0; chunk < kThreadChunks; ++chunk)
      *reinterpret_cast<uint4*>(staged + 8 * chunk) = weight_in[chunk];
#pragma unroll
    for (int h = 0; h < kStageProducts; ++h) row_bits[buffer][thread][h] = bits_in[h];
    __syncthreads();
    if (stage + 1 < stages) fetch_stage(stage + 1);  // in flight during the products
#pragma unroll
    for (int h = 0; h < kStageProducts; ++h) {
      v4u b_operand[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        b_operand[j] = *reinterpret_cast<const v4u*>(
            &weight_tile[buffer][(16 * j + li) * kProjectWeightPitch + kProjectStep * h + 8 * lg]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint2 bits = row_bits[buffer][wave * 64 + 16 * i + li][h];
        const uint32_t byte = (bits.x >> (8 * lg)) & 0xffu;
        const uint32_t valid = (bits.y >> (8 * lg)) & 1u;  // a head is valid as a whole
        const uint2 low = *reinterpret_cast<const uint2*>(
            ternary_table + 2 * ((valid << 4) | (byte & 15u)));
        const uint2 high = *reinterpret_cast<const uint2*>(
            ternary_table + 2 * ((valid << 4) | (byte >> 4)));
        const v4u a_operand = {low.x, low.y, high.x, high.y};
        // (the weights as the row operand: a lane then holds four neighbouring output
        // columns of one token, which leave as one 8-byte store)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma_bf16(b_operand[j], a_operand, acc[i][j]);
      }
    }
  }
  // lane (li, lg) holds columns 4 lg .. 4 lg + 3 of every 16-column tile for token li of
  // every 16-token tile
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t token = row0 + wave * 64 + 16 * i + li;
    if (token >= P.tokens) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t index = token * P.N + n0 + 16 * j + 4 * lg;
      v4f value = acc[i][j];
      if (P.residual != nullptr) {
        const uint2 added = *reinterpret_cast<const uint2*>(P.residual + index);
        value[0] += __uint_as_float(added.x << 16);
        value[1] += __uint_as_float(added.x & 0xffff0000u);
        value[2] += __uint_as_float(added.y << 16);
        value[3] += __uint_as_float(added.y & 0xffff0000u);
      }
      *reinterpret_cast<uint2*>(P.out + index) =
          make_uint2(bf16_nearest(value[0]) | (bf16_nearest(value[1]) << 16),
                     bf16_nearest(value[2]) | (bf16_nearest(value[3]) << 16));
    }
  }
}

int forward_entry(const rosa_problem* problem, const void* query, const void* key,
                  const void* value, void* output, int32_t* packed_query, int32_t* packed_key,
                  int32_t* routes, int32_t* lengths, void* workspace, size_t workspace_bytes,
                  void* stream, uint32_t* sign_words, uint8_t* routed, bool words_given = false,
                  bool allow_index = true) {
  ProblemView view;
  const int bad = check_problem(problem, &view);
  if (bad != 0) return bad;
  if ((!words_given && (!query || !key)) || !value || !packed_query || !packed_key || !workspace)
    return fail(2, "hard_forward: NULL tensor or workspace pointer");
  if (workspace_bytes < carve_forward(view, allow_index).total)
    return fail(3, "hard_forward: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (problem->dtype) {
    case ROSA_DTYPE_F32:
      return run_forward<ROSA_DTYPE_F32>(problem, view, query, key, value, output, packed_query,
                                         packed_key, routes, lengths, workspace, s, sign_words,
                                         routed, words_given, allow_index);
    case ROSA_DTYPE_F16:
      return run_forward<ROSA_DTYPE_F16>(problem, view, query, key, value, output, packed_query,
                                         packed_key, routes, lengths, workspace, s, sign_words,
                                         routed, words_given, allow_index);
    default:
      return run_forward<ROSA_DTYPE_BF16>(problem, view, query, key, value, output, packed_query,
                                          packed_key, routes, lengths, workspace, s, sign_words,
                                          routed, words_given, allow_index);
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

// The router's index of the keys in the caller's workspace: bucket offsets, routes by bucket,
// one byte per run and one per block of the routing grid.
struct RouterWorkspace {
  size_t bucket_begin, bucket_routes, run_scan, left_over, total;
  int blocks_per_run;
};

// Updates the index is used for: symbols of six bits or more (as in the training forward),
// chunks beyond the per-row kernel's, and histories long enough for the extra launches to pay.
constexpr int kRouterIndexLongestMin = 512;

bool router_index_suits(const rosa_router_update& u) {
  return u.qk_bits >= kIndexSymbolBitsMin && u.longest_chunk > kRouterDecodeRows &&
         u.longest_total >= kRouterIndexLongestMin;
}

RouterWorkspace carve_router(const rosa_router_update& u) {
  RouterWorkspace w;
  const size_t runs = static_cast<size_t>(u.S) * u.H;
  w.blocks_per_run = (u.longest_chunk + kWave - 1) / kWave;
  size_t cursor = 0;
  w.bucket_begin = cursor; cursor += align_up(sizeof(int32_t) * runs * ((size_t(1) << u.qk_bits) + 1));
  w.bucket_routes = cursor;
  cursor += align_up(sizeof(uint2) * runs * static_cast<size_t>(std::max(u.longest_total, 1)));
  w.run_scan = cursor; cursor += align_up(runs);
  w.left_over = cursor; cursor += align_up(runs * static_cast<size_t>(std::max(w.blocks_per_run, 1)));
  w.total = cursor;
  return w;
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
  // the kernel moves 16 bytes of a weight row or of four heads' words, and 8 bytes of an
  // output row, per access
  const auto misaligned = [](const void* pointer, uintptr_t bytes) {
    return (reinterpret_cast<uintptr_t>(pointer) & (bytes - 1)) != 0;
  };
  if (misaligned(weight, 16) || misaligned(sign_words, 16) || misaligned(routed, 4) ||
      misaligned(out, 8) || misaligned(residual, 8))
    return fail(1, "project_routed_bits: weight and sign_words must be 16-byte aligned, out and "
                   "residual 8-byte, routed 4-byte");
  const dim3 grid(static_cast<unsigned>(row_blocks), static_cast<unsigned>(N / kProjectColumns));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (Dv == 8) {
    hipLaunchKernelGGL(project_routed_bits_kernel<4>, grid, dim3(256), 0, s, P);
  } else if (Dv == 16) {
    hipLaunchKernelGGL(project_routed_bits_kernel<2>, grid, dim3(256), 0, s, P);
  } else {
    hipLaunchKernelGGL(project_routed_bits_kernel<0>, grid, dim3(256), 0, s, P);
  }
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
  // the index of the keys (16 more bytes per token and head) is used where it fits as well
  const bool with_index = carve_forward(view, true).total <= kStaticScratchBytes;
  if (carve_forward(view, with_index).total > kStaticScratchBytes) {
    return fail(3, "hard_forward_static: the problem needs more than the 16 MiB of static "
                   "scratch (4 bytes per token and head); use rosa_hip_hard_forward");
  }
  void* address = nullptr;
  const int status = static_scratch_address(&address);
  if (status != 0) return status;
  return forward_entry(problem, query, key, value, output, packed_query, packed_key, routes,
                       nullptr, address, kStaticScratchBytes, stream, nullptr, nullptr, false,
                       with_index);
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

size_t rosa_hip_router_workspace_bytes(const rosa_router_update* update) {
  if (update == nullptr || update->S < 1 || update->H < 1 || update->qk_bits < 1 ||
      update->qk_bits > 8 || update->longest_chunk < 0 || update->longest_total < 0)
    return 0;
  return router_index_suits(*update) ? carve_router(*update).total : 0;
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
  U.history_lengths_out = u.history_lengths_out;
  U.query_history = u.query_history;
  U.key_history = u.key_history;
  U.payload_history = u.payload_history;
  U.query = u.query; U.key = u.key; U.payload = u.payload;
  U.output = u.output;
  U.matched_key_end = u.matched_key_end;
  U.tokens = u.tokens;
  U.blocks_per_run = 1;
  U.bucket_begin = nullptr; U.bucket_routes = nullptr; U.run_scan = nullptr; U.left_over = nullptr;
  U.index_stride = 0; U.log_buckets = 0; U.budget_base = 0;
  const int index_mode = g_forward_index_mode.load(std::memory_order_relaxed);
  bool indexed = false;
  if (u.workspace != nullptr && index_mode != 1 && router_index_suits(u)) {
    if (u.longest_total > u.capacity)
      return fail(1, "router: longest_total exceeds the capacity of a run");
    const RouterWorkspace w = carve_router(u);
    if (u.workspace_bytes < w.total) return fail(3, "router: workspace too small");
    U.bucket_begin = at<int32_t>(u.workspace, w.bucket_begin);
    U.bucket_routes = at<uint2>(u.workspace, w.bucket_routes);
    U.run_scan = at<uint8_t>(u.workspace, w.run_scan);
    U.left_over = at<uint8_t>(u.workspace, w.left_over);
    U.index_stride = std::max(u.longest_total, 1);
    U.log_buckets = u.qk_bits;
    U.budget_base = index_mode == 2 ? -(1 << 30) : 64;
    indexed = true;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t symbols = static_cast<int64_t>(u.tokens) * u.H;
  const int64_t runs = static_cast<int64_t>(u.S) * u.H;
  const bool decode = u.longest_chunk > 0 && u.longest_chunk <= kRouterDecodeRows;
  if (decode && u.history_lengths_out != nullptr) {
    // a decoding step with the lengths going to an array of their own: one launch
    U.blocks_per_run = u.longest_chunk;
    const int64_t blocks = runs * U.blocks_per_run;
    if (blocks > INT32_MAX) return fail(1, "router: slots * heads * row blocks must fit in int32");
    hipLaunchKernelGGL(router_decode_step_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWave),
                       0, s, U);
  } else {
    hipLaunchKernelGGL(router_append_kernel, dim3(blocks_for(symbols, 256)), dim3(256), 0, s, U);
    if (u.longest_chunk > 0) {
      U.blocks_per_run = decode ? u.longest_chunk : (u.longest_chunk + kWave - 1) / kWave;
      const int64_t blocks = runs * U.blocks_per_run;
      if (blocks > INT32_MAX) return fail(1, "router: slots * heads * row blocks must fit in int32");
      if (decode) {
        hipLaunchKernelGGL(router_decode_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWave),
                           0, s, U);
      } else {
        if (indexed) {
          hipLaunchKernelGGL(router_index_kernel, dim3(static_cast<unsigned>(runs)),
                             dim3(kIndexThreads), 0, s, U);
          hipLaunchKernelGGL(router_candidates_kernel, dim3(static_cast<unsigned>(blocks)),
                             dim3(kWave), 0, s, U);
        }
        hipLaunchKernelGGL(router_route_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWave),
                           0, s, U);
      }
    }
    hipLaunchKernelGGL(router_advance_kernel, dim3(blocks_for(u.S, 256)), dim3(256), 0, s, U);
  }
  const hipError_t status = hipGetLastError();
  if (status != hipSuccess) return fail_hip(status, "router launch");
  return 0;
}

void rosa_hip_set_gradient_block_waves(int waves) {
  g_gradient_block_waves = (waves == 1 || waves == 2) ? waves : 0;
}

void rosa_hip_set_gradient_piece_rows(int rows) { g_gradient_piece_rows = rows < -1 ? 0 : rows; }

void rosa_hip_set_forward_index(int mode) { g_forward_index_mode = (mode >= 1 && mode <= 3) ? mode : 0; }

void rosa_hip_set_record_budget(size_t bytes) {
  g_record_budget_bytes = bytes;  // (size_t)-1: the default
}

int rosa_hip_stage_timing(int enable) {
  if (enable && !g_timer.created) {
    for (int i = 0; i < kStageCount; ++i) {
      for (int slot = 0; slot < kStageRing; ++slot) {
        if (hipEventCreate(&g_timer.begin[i][slot]) != hipSuccess ||
            hipEventCreate(&g_timer.end[i][slot]) != hipSuccess)
          return fail(5, "hipEventCreate failed");
      }
    }
    g_timer.created = true;
  }
  for (int i = 0; i < kStageCount; ++i) g_timer.runs[i] = 0;
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
    if (g_timer.runs[i] == 0) continue;
    const int slot = static_cast<int>((g_timer.runs[i] - 1) % kStageRing);
    if (hipEventSynchronize(g_timer.end[i][slot]) != hipSuccess) return fail(5, "event sync failed");
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, g_timer.begin[i][slot], g_timer.end[i][slot]) != hipSuccess)
      return fail(5, "event elapsed failed");
    milliseconds[i] = ms;
  }
  return 0;
}

int rosa_hip_stage_totals(float* milliseconds, int* runs, int count) {
  if (!g_timer.created) return fail(5, "stage timing was never enabled");
  if (!milliseconds || !runs) return fail(2, "stage_totals: NULL pointer");
  for (int i = 0; i < count && i < kStageCount; ++i) {
    const int kept = static_cast<int>(std::min<int64_t>(g_timer.runs[i], kStageRing));
    double total = 0.0;
    for (int back = 1; back <= kept; ++back) {
      const int slot = static_cast<int>((g_timer.runs[i] - back) % kStageRing);
      if (hipEventSynchronize(g_timer.end[i][slot]) != hipSuccess) return fail(5, "event sync failed");
      float ms = 0.0f;
      if (hipEventElapsedTime(&ms, g_timer.begin[i][slot], g_timer.end[i][slot]) != hipSuccess)
        return fail(5, "event elapsed failed");
      total += ms;
    }
    milliseconds[i] = static_cast<float>(total);
    runs[i] = kept;
    g_timer.runs[i] = 0;
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

int rosa_hip_gradient_piece_plan(const rosa_problem* problem, int* piece_rows, int* pieces) {
  ProblemView view;
  const int status = check_problem(problem, &view);
  if (status != 0) return status;
  const int slice_width = std::min(view.L.Dv, kValueSlice);
  const int dvp = padded_value_width(slice_width);
  const int symbol_tiles = view.L.D > 16 ? 2 : 1;
  const int64_t units = static_cast<int64_t>(view.L.slots) * view.L.H;
  const GradientBlockPlan blocks = plan_gradient_blocks(
      dvp, view.L.D, value_words(slice_width), grad_term_pitch(view.grad_terms, dvp), units);
  PiecePlan plan{0, 1};
  if (blocks.waves == 1) {
    plan = plan_band_pieces(units, view.L.varlen ? view.L.N : view.L.T, view.L.W,
                            resident_gradient_waves((dvp + 15) / 16, symbol_tiles),
                            gradient_segment(dvp));
  }
  if (piece_rows != nullptr) *piece_rows = plan.piece_rows;
  if (pieces != nullptr) *pieces = plan.max_pieces;
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
  const int waves = max_resident_blocks(), tiles = 2000;
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
