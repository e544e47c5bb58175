#include "attention_plan.h"

#include <algorithm>
#include <vector>

namespace liyab_host {

void attn_counts(int n_seqs, const int* q_lens, int decode_q_len, int attn_tile, int* n_tiles, int* n_single) {
    int tiles = 0, single = 0;
    for (int i = 0; i < n_seqs; ++i) {
        if (q_lens[i] <= decode_q_len) single += q_lens[i];
        else tiles += (q_lens[i] + attn_tile - 1) / attn_tile;
    }
    *n_tiles = tiles;
    *n_single = single;
}

void attn_fill(int n_seqs, const int* q_lens, const int* first_pos, int decode_q_len, int attn_tile, int32_t* words) {
    struct Tile {
        int seq, row, pos, count;
    };
    int n_tiles = 0, n_single = 0;
    attn_counts(n_seqs, q_lens, decode_q_len, attn_tile, &n_tiles, &n_single);
    std::vector<Tile> tiles;
    tiles.reserve(static_cast<size_t>(n_tiles));
    int32_t* work = words;
    int32_t* single = words + 4 * std::max(n_tiles, 1);
    work[0] = work[1] = work[2] = work[3] = 0;
    single[0] = 0;
    int row0 = 0, k = 0;
    for (int i = 0; i < n_seqs; ++i) {
        const int n = q_lens[i], first = first_pos[i];
        if (n <= decode_q_len) {
            for (int j = 0; j < n; ++j) single[k++] = row0 + j;
        } else {
            for (int t0 = 0; t0 < n; t0 += attn_tile) tiles.push_back({i, row0 + t0, first + t0, std::min(attn_tile, n - t0)});
        }
        row0 += n;
    }
    // a tile's work grows with its last position: the longest first, so that the short ones
    // fill the gaps at the end
    std::stable_sort(tiles.begin(), tiles.end(), [](const Tile& a, const Tile& b) { return a.pos + a.count > b.pos + b.count; });
    for (size_t t = 0; t < tiles.size(); ++t) {
        work[4 * t] = tiles[t].seq;
        work[4 * t + 1] = tiles[t].row;
        work[4 * t + 2] = tiles[t].pos;
        work[4 * t + 3] = tiles[t].count;
    }
}

}  // namespace liyab_host
