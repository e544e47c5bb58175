// Attention's own words of a step's metadata: nothing in the step's common block (step_meta.h) or in
// the cache manager knows of them; the attention part's step planner (parts/attention.py) asks for them
// through the C interface and lays them behind the common block, as any part's planner may with words of
// its own. They are laid out natively because a prompt's step names hundreds of tiles.
#pragma once

#include <cstdint>

namespace liyab_host {

// Attention's own words of a step in which some request brings more than decode_q_len tokens:
// the long portions cut into tiles of up to attn_tile consecutive queries (4 words a tile: request
// index, first row, first position, queries; the tile that ends at the latest position first, so
// that the short ones fill the gaps at the end), and the rows of the short portions, which are
// attended one by one. attn_counts gives (tiles, single rows); attn_fill writes 4 * max(tiles, 1)
// words of tiles followed by max(single rows, 1) words of rows. first_pos: each request's length
// before the step.
void attn_counts(int n_seqs, const int* q_lens, int decode_q_len, int attn_tile, int* n_tiles, int* n_single);
void attn_fill(int n_seqs, const int* q_lens, const int* first_pos, int decode_q_len, int attn_tile, int32_t* words);

}  // namespace liyab_host
