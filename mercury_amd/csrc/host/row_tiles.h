// Row tiles of a step: the rows of a sequence are its (token, head-in-group) pairs, `group`
// per token; a tile is `tile_rows` consecutive rows of one sequence.
#pragma once

#include <vector>

namespace mercury {

int count_tiles(const std::vector<int>& counts, int group, int tile_rows);
// tile_seq and tile_row0, appended to `seq` and `row0`.
void build_tiles(const std::vector<int>& counts, int group, int tile_rows, std::vector<int>& seq,
                 std::vector<int>& row0);

}  // namespace mercury
