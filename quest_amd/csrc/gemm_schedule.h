// How the persistent large-tile GEMM kernels (gemm_big.hip, gemm_e2m3.hip) divide the output among their workgroups:
// cells of 256 tokens x 32 channels ("units"), eight groups of workgroups (one per XCD and its L2 when the grid
// allows), and per workgroup a contiguous run of cells that it walks in tiles of up to MAXU units.
#pragma once
#include "gemm_tiles.h"

namespace quest {

struct Schedule {
    int tiles_t;        // token tiles of 256
    int units;          // channel units of 32
    int groups;         // channel super-groups (one per XCD when the grid allows)
    int row_tiles;      // > 0: one tile per workgroup, this many per token tile of a group (0: contiguous runs of cells)
    int by_tokens;      // how many ways the groups divide the token tiles (1: every group takes all token tiles and 1/groups of the
                        // channel units; groups: the other way round; in between: a groups_t x groups / groups_t grid of groups)
};

struct Cursor {          // walks a workgroup's run of cells tile by tile, stage by stage (no divisions)
    int tt, u;               // next cell: token tile, channel unit inside the group
    int left;                // cells left in the run
    int nug, ug0;
    int tok0, ch0, width;    // current tile
    int kt;                  // next stage of the current tile
    bool valid;
};

template <int MAXU>
__device__ __forceinline__ void cursor_next_tile(Cursor &c) {
    if (c.left <= 0) { c.valid = false; return; }             // keeps pointing at the last tile
    int width = c.nug - c.u;
    width = width < c.left ? width : c.left;
    // kept in a scalar register: two chained minima would otherwise be selected as the vector ALU's three-operand
    // minimum, which drags the whole cursor into vector registers (and those get spilled at the register peaks)
    asm volatile("" : "+s"(width));
    width = width < MAXU ? width : MAXU;
    c.tok0 = c.tt * kBigTileRows;
    c.ch0 = (c.ug0 + c.u) * 32;
    c.width = width;
    c.kt = 0;
    c.valid = true;
    c.left -= width;
    c.u += width;
    if (c.u == c.nug) { c.u = 0; c.tt++; }
}

// The run of cells of workgroup blockIdx.x, as a cursor in front of its first tile (the caller then steps it with
// cursor_next_tile).  Everything is wave-uniform and brought back to scalar registers.
__device__ __forceinline__ void cursor_begin(const Schedule &sch, Cursor &cc) {
    const int rank = __builtin_amdgcn_readfirstlane((int)(blockIdx.x / sch.groups));
    const int grp = blockIdx.x - rank * sch.groups;
    const int per_grp = __builtin_amdgcn_readfirstlane((int)(gridDim.x / sch.groups));
    // A group (= an XCD and its L2 when there are eight) owns a slice of the channel units and all token tiles, or --
    // by_tokens -- a slice of the token tiles and all units: whichever operand is the smaller one is then the one every
    // XCD fetches whole (and keeps in its L2), and the larger one is fetched once in total.
    int ug0 = 0, ug1 = sch.units, tt_lo = 0, tt_hi = sch.tiles_t;
    {
        const int gt_n = sch.by_tokens > 0 ? sch.by_tokens : 1;          // groups along the tokens
        const int gu_n = sch.groups / gt_n;                              // groups along the channels
        const int gt = grp % gt_n, gu = grp / gt_n;
        if (gt_n > 1) {
            tt_lo = __builtin_amdgcn_readfirstlane((int)(((long)gt * sch.tiles_t) / gt_n));
            tt_hi = __builtin_amdgcn_readfirstlane((int)(((long)(gt + 1) * sch.tiles_t) / gt_n));
        }
        if (gu_n > 1) {
            ug0 = __builtin_amdgcn_readfirstlane((int)(((long)gu * sch.units) / gu_n));
            ug1 = __builtin_amdgcn_readfirstlane((int)(((long)(gu + 1) * sch.units) / gu_n));
        }
    }
    cc.nug = ug1 - ug0;
    cc.ug0 = ug0;
    // the divisions run on the vector ALU (there is no scalar divide); readfirstlane brings the (uniform) results
    // back to scalar registers, and with them the whole cursor arithmetic of the tile loop
    const long cells = (long)(tt_hi - tt_lo) * cc.nug;
    int pos0, pos1;
    if (sch.row_tiles > 0) {
        // about one tile per workgroup: every token tile's units are cut into row_tiles tiles of equal width (+-1) and
        // workgroup `rank` takes one of them.  An even split of the cells would let runs cross token-tile boundaries,
        // and a workgroup with two tiles (each a full K loop) then takes twice as long as the others.
        const int q = sch.row_tiles;
        const int tile_t = __builtin_amdgcn_readfirstlane(rank / q);
        const int i = rank - tile_t * q;
        pos0 = tile_t * cc.nug + __builtin_amdgcn_readfirstlane((i * cc.nug) / q);
        pos1 = tile_t * cc.nug + __builtin_amdgcn_readfirstlane(((i + 1) * cc.nug) / q);
        if (tile_t >= sch.tiles_t) pos1 = pos0;
    } else {
        pos0 = __builtin_amdgcn_readfirstlane((int)((cells * rank) / per_grp));
        pos1 = __builtin_amdgcn_readfirstlane((int)((cells * (rank + 1)) / per_grp));
    }
    const int tt_rel = __builtin_amdgcn_readfirstlane(pos0 / cc.nug);
    cc.tt = tt_lo + tt_rel;
    cc.u = pos0 - tt_rel * cc.nug;
    cc.left = pos1 - pos0;
    cc.valid = false;
    cc.tok0 = cc.ch0 = cc.width = cc.kt = 0;
}

// Host side: the schedule and the grid for M tokens x N channels with tiles of up to max_units units and
// wg_per_cu persistent workgroups on each of the device's `cus` compute units.
inline Schedule make_schedule(int M, int N, int max_units, int wg_per_cu, int cus, long *grid_out, int tok_split = 0) {
    Schedule sch;
    sch.tiles_t = (M + kBigTileRows - 1) / kBigTileRows;
    sch.units = (N + 31) / 32;
    const long cells = (long)sch.tiles_t * sch.units;
    long grid = (long)wg_per_cu * cus;                         // persistent: one or two workgroups per CU
    if (grid > cells) grid = cells;
    sch.groups = (grid % 8 == 0 && sch.units >= 8) ? 8 : 1;
    sch.row_tiles = 0;
    sch.by_tokens = 0;
    // More tokens than channels: the eight XCD groups divide the token tiles instead of the channel units, so that the
    // weights (the smaller operand) are what every XCD fetches whole and the activation codes cross the fabric once
    // (measured +4..7 % at M = 16384 with N = 1024..5632; no difference at M = 4096, N = 11008 either way).
    if (M > N && grid % 8 == 0 && sch.tiles_t >= 8) {
        sch.groups = 8;
        sch.by_tokens = 8;
    }
    // tok_split < 0: the grid of groups (1 x 8, 2 x 4, 4 x 2 or 8 x 1) that fetches least from behind the L2s.  The
    // workgroups of a group work on T token tiles x C channel ranges at a time (T C = workgroups per group) and one such
    // round fetches T + C operand tiles of equal size; splitting the token tiles g ways makes T = tiles_t / g.  At
    // M = 4096, N = 11008: 16 + 2 tiles as 1 x 8, 8 + 4 as 2 x 4 (a third less traffic, the same time); at M = 8192:
    // 32 + 1 against 8 + 4 as 4 x 2 (238 -> 217 us).  Only where every workgroup has several full tiles to walk.
    if (tok_split < 0 && grid % 8 == 0 && sch.units >= 8 && cells >= 2L * max_units * grid) {
        const long per_grp = grid / 8;
        long best_cost = 0;
        int best = 0;
        for (int g = 1; g <= 8; g *= 2) {
            if (sch.tiles_t % g != 0 || sch.units < (long)max_units * (8 / g)) continue;
            long t = sch.tiles_t / g;
            if (t > per_grp) t = per_grp;
            const long c = per_grp / t > 1 ? per_grp / t : 1;
            if (best == 0 || t + c < best_cost) { best = g; best_cost = t + c; }
        }
        if (best > 0) {
            sch.groups = 8;
            sch.by_tokens = best > 1 ? best : 0;
        }
    } else if (!sch.by_tokens && sch.groups == 8 && tok_split > 1 && sch.tiles_t % tok_split == 0 &&
               sch.units >= 2L * max_units * (8 / tok_split) && cells >= 2L * max_units * grid) {
        sch.by_tokens = tok_split;
    }
    if (!sch.by_tokens) {
        // few cells per workgroup: one tile each, cut along the channel units of single token tiles (see cursor_begin)
        const long per_grp = grid / sch.groups;
        const int nug = (sch.units + sch.groups - 1) / sch.groups;
        if ((long)sch.tiles_t * nug <= (long)max_units * per_grp) {
            for (int w = 1; w <= max_units; w++) {
                const int q = (nug + w - 1) / w;
                if ((long)sch.tiles_t * q <= per_grp) {
                    sch.row_tiles = q;
                    grid = (long)sch.groups * sch.tiles_t * q;
                    break;
                }
            }
        }
    }
    *grid_out = grid;
    return sch;
}

}  // namespace quest
