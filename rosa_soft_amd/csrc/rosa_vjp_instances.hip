// The band kernels of the surrogate backward for ONE tile family, compiled once per family
// with -DROSA_FAMILY_NVW (sign words per value column), -DROSA_FAMILY_DVP (padded value
// width) and -DROSA_FAMILY_DT (symbol tiles), so that the families build side by side.
// The library's main translation unit launches the kernels through the table exported here.

#include "rosa_vjp_bands.hpp"

#ifndef ROSA_FAMILY_NVW
#define ROSA_FAMILY_NVW 1
#endif
#ifndef ROSA_FAMILY_DVP
#define ROSA_FAMILY_DVP 8
#endif
#ifndef ROSA_FAMILY_DT
#define ROSA_FAMILY_DT 1
#endif

namespace {

constexpr int NVW = ROSA_FAMILY_NVW;
constexpr int DVP = ROSA_FAMILY_DVP;
constexpr int DT = ROSA_FAMILY_DT;

static_assert((NVW == 1 && (DVP == 8 || DVP == 16 || DVP == 32)) || (NVW == 2 && DVP == 64),
              "tile families: widths 8, 16, 32 with one sign word, 64 with two");
static_assert(DT == 1 || DT == 2, "one or two symbol tiles");
// At most 64 KB of dynamic LDS per block: what every kernel may use without raising its
// limit first.  (Raising it would be a configuration call per launch, and those are
// refused while a stream is being captured into a graph.)
static_assert((gradient_wave_floats(DVP, grad_term_pitch(kMaxGradTerms, DVP)) +
               gradient_shared_fixed_floats(gradient_segment(DVP), NVW, 1)) * sizeof(float) <=
                  64 * 1024,
              "dynamic LDS of the gradient kernel");

template <typename Kernel>
const void* address_of(Kernel kernel) { return reinterpret_cast<const void*>(kernel); }

template <bool VARLEN, bool DROPOUT>
void fill_layout(const void** table) {
  constexpr int v = VARLEN ? 1 : 0, d = DROPOUT ? 1 : 0;
  if constexpr (DT == 1) {
    // the row kernels do not depend on the symbol tiles: they live in the one-tile family
    table[vjp_kernel_slot_row_max(v)] = address_of(vjp_row_max_kernel<NVW, VARLEN>);
    table[vjp_kernel_slot_row_stats(v, d)] =
        address_of(vjp_row_stats_kernel<NVW, DVP, VARLEN, DROPOUT>);
  }
  table[vjp_kernel_slot_gradients(v, d, kGradientFormOneWave, 2)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 2, false>);
  table[vjp_kernel_slot_gradients(v, d, kGradientFormOneWave, 3)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 3, false>);
  table[vjp_kernel_slot_gradients(v, d, kGradientFormTwoWaves, 2)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 2, 2, false>);
  table[vjp_kernel_slot_gradients(v, d, kGradientFormTwoWaves, 3)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 2, 3, false>);
  table[vjp_kernel_slot_gradients(v, d, kGradientFormPieces, 2)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 2, true>);
  table[vjp_kernel_slot_gradients(v, d, kGradientFormPieces, 3)] =
      address_of(vjp_gradients_kernel<NVW, DVP, DT, VARLEN, DROPOUT, 1, 3, true>);
}

const void* const* family_table() {
  static const void* table[kVjpKernelSlots] = {};
  static const bool filled = [] {
    fill_layout<false, false>(table);
    fill_layout<false, true>(table);
    fill_layout<true, false>(table);
    fill_layout<true, true>(table);
    return true;
  }();
  (void)filled;
  return table;
}

}  // namespace

#define ROSA_FAMILY_PASTE(nvw, dvp, dt) rosa_vjp_kernels_##nvw##_##dvp##_##dt
#define ROSA_FAMILY_SYMBOL(nvw, dvp, dt) ROSA_FAMILY_PASTE(nvw, dvp, dt)

extern "C" const void* const* ROSA_FAMILY_SYMBOL(ROSA_FAMILY_NVW, ROSA_FAMILY_DVP,
                                                 ROSA_FAMILY_DT)(void) {
  return family_table();
}
