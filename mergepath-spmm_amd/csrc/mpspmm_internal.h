// Shapes shared by the host and device halves of the library (not installed).
#ifndef MPSPMM_INTERNAL_H
#define MPSPMM_INTERNAL_H

// How one 64-lane wavefront is cut into lane-groups for feature width K.
// A lane-group walks one merge-path partition (or one row / one nonzero
// group in the comparison kernels); each of its lanes owns `vec` adjacent
// output columns.
struct mps_lane_shape {
    int vec;         // columns per lane: 16 bytes worth (4 fp32 / 8 fp16), 4 fp16 for narrow rows, or 1
    int lanes_log2;  // log2(lanes per group), lanes in 4..64
    int groups;      // lane-groups per wavefront = 64 / lanes
    int col_tiles;   // passes over the columns when K > lanes * vec
};

static inline mps_lane_shape mps_make_lane_shape(int K, int elem_bytes)
{
    mps_lane_shape s;
    int vec = 16 / elem_bytes;
    if (!(K % vec == 0 && K >= 4 * vec)) vec = (K % 4 == 0 && K >= 16) ? 4 : 1;  // fp16, K = 16 .. 28: 8 bytes per lane
    int want = (K + vec - 1) / vec;
    int l2 = 2;
    while ((1 << l2) < want && l2 < 6) ++l2;
    s.vec = vec;
    s.lanes_log2 = l2;
    s.groups = 64 >> l2;
    int per_tile = (1 << l2) * vec;
    s.col_tiles = (K + per_tile - 1) / per_tile;
    return s;
}

#endif
