// Fixed-order sums for the pieces of long rows of the forward pass (row_pieces.hip).
#ifndef E3J_AMD_CSRC_ROW_PIECES_H_
#define E3J_AMD_CSRC_ROW_PIECES_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace e3j_amd {

// Bytes of the caller's `partials` buffer: max_segments rows of row_floats floats, then the list
// the piece launch reads (4 + 3 * max_segments int32, pieces numbered instead of named by row).
size_t row_partials_bytes(int64_t max_segments, int64_t row_floats);
// The int32 list behind the rows of `partials`.
int32_t *row_partials_list(float *partials, int64_t max_segments, int64_t row_floats);
// Before the piece launch: list[i] = (i, begin, end) of piece i, rows 0 .. count-1 of partials zeroed.
int launch_prepare_partials(const int32_t *segments, int32_t max_segments, int64_t row_floats, float *partials,
                            hipStream_t stream);
// After it: out[row] += partials[i] for the pieces of every row, in list order (pieces of one row
// are adjacent and in position order, the first of them row_piece positions behind the row's
// start: e3j_amd_row_segments_build).
int launch_combine_pieces(const int32_t *segments, const int32_t *row_ptr, int32_t max_segments, int32_t row_piece,
                          int64_t row_floats, const float *partials, float *out, hipStream_t stream);

}  // namespace e3j_amd
#endif
