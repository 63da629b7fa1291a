// Order in which workgroup ids walk the output tiles of the tiled GEMM.  The same arithmetic as the reference's
// xcd_remap_bx_by (kernels/common/mma/mfma_preshuffle_pipeline.py:685-729) with linear id = bx*gx + by:
// the hardware deals consecutive workgroup ids round-robin over the 8 XCDs, so id -> (xcd = id % 8, in_xcd = id / 8)
// is first turned into a contiguous range of work per XCD, and that range then walks the tiles in groups of
// `group_m` M-tiles per sweep over N (column-major inside a group), so the A and W panels one XCD touches at a time
// stay in its L2.  Host and device use this one function.
#pragma once

#if defined(__HIPCC__)
#define PSG_HD __host__ __device__
#else
#define PSG_HD
#endif

PSG_HD inline void psg_tile_order(int id, int tiles_m, int tiles_n, int group_m, int* tm, int* tn) {
    const int num = tiles_m * tiles_n;
    const int q = num >> 3, r = num & 7;
    const int xcd = id & 7, in_xcd = id >> 3;
    const int wg = xcd * q + (xcd < r ? xcd : r) + in_xcd;
    const int per_group = group_m * tiles_n;
    const int g = wg / per_group;
    const int first_m = g * group_m;
    const int size_m = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_g = wg - g * per_group;
    *tm = first_m + in_g % size_m;
    *tn = in_g / size_m;
}
