// GEMM core for prefill-sized M on the FP6 matrix cores: a third route beside the popcount and
// int8 MFMA strategies, for operands that fit a 6-bit float exactly.
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for every bit pair whose operands are
// unsigned of at most 4 bits or signed of at most 5 bits (w2a2 ... w5a5 signed, w2a2 ... w4a4
// unsigned, w2a4).
//
// Why it is exact.  CDNA4's v_mfma_f32_32x32x64_f8f6f4 multiplies FP6 (E2M3: sign, 2 exponent
// bits, 3 mantissa bits) operands at twice the int8 rate and accumulates in fp32.  Read with
// 1/8 as the unit, the E2M3 codes 0..15 of the subnormal range and the first binade are the
// integers 0..15 in plain binary, and 16 is 0b010000: a sign-magnitude integer of magnitude
// <= 16 IS its FP6 encoding.  Every product is a multiple of 1/64 and every partial sum is
// below 2^24 units as long as max|x| * max|w| * K < 2^24 (checked by the host), so the fp32
// accumulation never rounds and acc * 64 is the integer result, bit for bit.
//
// Operand format (library-private, written by relayout_planes_fp6_kernel): a row's K tile of 128
// elements is one record of 96 bytes = four 192-bit strings of 32 six-bit codes; strings 0 and 1
// feed lanes 0-31 of the two MFMA K steps of the tile, strings 2 and 3 lanes 32-63, so a lane
// fetches both steps with three aligned ds_read_b128.  Records are stored tiled[kt][row][96 B].
//
// The kernel itself is the format-generic staged kernel of abq_gemm_staged.h (tiles loaded straight
// into LDS, nothing unpacked); this file instantiates it for the FP6 records.
#include "abq_gemm_staged.h"

namespace abq {

// Tile space: MFMA tiles per wave (TM, TN) and waves along M, N; nstage 5 marks the FP6 records.
#define ABQ_FP6_VARIANTS(V) V(2, 2, 4, 2) V(4, 2, 2, 2) V(2, 2, 2, 2) V(2, 1, 2, 2) V(1, 1, 2, 2)
#define ABQ_FP6_ENTRY(TM, TN, WM, WN)                                                             \
    { 32, TM, TN, WM, WN, 1, 5, &launch_mfma_staged<6, 6, true, true, TM, TN, WM, WN>, 128,       \
      StagedStages<6, 6, true, TM, TN, WM, WN>::kLds },
static const KernelEntry kFp6Entries[] = { ABQ_FP6_VARIANTS(ABQ_FP6_ENTRY) };

const KernelEntry *fp6_entries(int *count)
{
    *count = (int)(sizeof(kFp6Entries) / sizeof(kFp6Entries[0]));
    return kFp6Entries;
}

// The same tiles with group scales (groups of 128), where a wave has at least two MFMA tiles.
#define ABQ_FP6_GROUPED_VARIANTS(V) V(2, 2, 4, 2) V(2, 2, 2, 2) V(2, 1, 2, 2)
#define ABQ_FP6_GENTRY(TM, TN, WM, WN)                                                                   \
    { 32, TM, TN, WM, WN, 1, 5, &launch_mfma_staged<6, 6, true, true, TM, TN, WM, WN, true>, 128,        \
      StagedStages<6, 6, true, TM, TN, WM, WN, true>::kLds },
static const KernelEntry kFp6GroupedEntries[] = { ABQ_FP6_GROUPED_VARIANTS(ABQ_FP6_GENTRY) };

const KernelEntry *fp6_grouped_entries(int *count)
{
    *count = (int)(sizeof(kFp6GroupedEntries) / sizeof(kFp6GroupedEntries[0]));
    return kFp6GroupedEntries;
}

} // namespace abq
