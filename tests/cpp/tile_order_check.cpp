// Host-only check of the work-item order of the large-tile kernel (blocked_tile_of, therock_amd/csrc/common.hpp):
// for every (row tiles, column tiles) pair the item numbers 0 .. rows * cols - 1 map onto every (column, row) pair
// exactly once, a full block's items are kTileRowBlock adjacent row tiles per column tile, and 32 consecutive items of
// a large expert span at most 4 row tiles and 9 column tiles (what one XCD holds at a time).  Exit code 0 = all hold.
#include <algorithm>
#include <cstdio>
#include <vector>

#include "../../therock_amd/csrc/common.hpp"

int main()
{
    using namespace mi355;
    for(int rows = 1; rows <= 130; rows++)
        for(int cols = 1; cols <= 40; cols++)
        {
            std::vector<int> seen(rows * cols, 0);
            for(int rel = 0; rel < rows * cols; rel++)
            {
                int col = -1, row = -1;
                blocked_tile_of(rel, rows, cols, col, row);
                if(col < 0 || col >= cols || row < 0 || row >= rows)
                {
                    std::printf("out of range: rows=%d cols=%d rel=%d -> col=%d row=%d\n", rows, cols, rel, col, row);
                    return 1;
                }
                seen[col * rows + row]++;
            }
            for(int v : seen)
                if(v != 1)
                {
                    std::printf("not a bijection: rows=%d cols=%d\n", rows, cols);
                    return 2;
                }
            if(rows >= 8 && cols >= 8) // (with fewer column tiles a block has fewer than 32 items)
                for(int start = 0; start + 32 <= (rows / kTileRowBlock * kTileRowBlock) * cols; start += 32)
                {
                    int rmin = rows, rmax = -1, cmin = cols, cmax = -1;
                    for(int rel = start; rel < start + 32; rel++)
                    {
                        int col, row;
                        blocked_tile_of(rel, rows, cols, col, row);
                        rmin = std::min(rmin, row); rmax = std::max(rmax, row);
                        cmin = std::min(cmin, col); cmax = std::max(cmax, col);
                    }
                    // one block: 4 row tiles x 8 column tiles; a chunk that straddles two blocks: 8 row tiles
                    if(rmax - rmin + 1 > 2 * kTileRowBlock || (rmax - rmin + 1 <= kTileRowBlock && cmax - cmin + 1 > 9))
                    {
                        std::printf("chunk too wide: rows=%d cols=%d start=%d spans %d rows x %d cols\n", rows, cols, start,
                                    rmax - rmin + 1, cmax - cmin + 1);
                        return 3;
                    }
                }
        }
    // an item number past the expert's items (a workgroup that finds no work reads an entry before it knows) divides by
    // nothing
    int col, row;
    blocked_tile_of(1000, 4, 3, col, row);
    std::printf("tile_order_check ok\n");
    return 0;
}
