// Internal interface of the table of measured best tiles (abq_tuning.hip).
#pragma once
#include "abq_gemm.h"

namespace abq {

struct TunedTile {
    abq_tile_config cfg;
    int M, N, K, group_size;
    float tops;
};

// abq_layout both operands of a tile are read in: ABQ_LAYOUT_FP6 (MMA 32x32x64), ABQ_LAYOUT_TILED (NSTAGE 4 and 6),
// else ABQ_LAYOUT_PLANES.  (A kernel on prepared layouts also takes operands still in planes and converts them into the
// caller's workspace; what counts for a lookup is the layout the weights are held in.)
int tile_operand_layout(const abq_tile_config &c);

// The fastest entry for this GEMM among those whose layout has its bit (1 << abq_layout) set in layout_mask; entries
// loaded at run time come before the compiled-in ones.
bool tuning_find(int x_bits, int w_bits, int is_signed, int M, int N, int K, int group, int layout_mask, TunedTile *out);

// A signed prefill-sized GEMM (more than 16 rows, no group scales) whose activations have 3, 5, 6 or 7 bits and whose
// weights have 2, 4 or 8: the library runs it as the pair (activations padded to the next width of one field, the same
// weights) when that pair has kernels on K-tiled records; the activations are converted per call anyway, the weight
// records are the pair's own (abq_api.hip).
bool activations_run_padded(int x_bits, int w_bits, int is_signed, int M, int group_size);

} // namespace abq
