// C entry points over index_math.h for the host-side replay tool (kernl_amd/debugger): the SAME functions the kernels
// are compiled from, built here with the host compiler only (g++ -shared -fPIC), no HIP involved.
#include "index_math.h"

using namespace kernl;

// Stream-K few-row linear kernel, 512 threads; (row blocks, units per stage) as the kernel is built: (1, 4), (2, 2),
// (4, 2), (8, 2).  which: 0 piece_unit(tid=a, i=b), 1 piece_row(tid=a, i=b), 2 piece_index(tid=a), 3 piece_dst(tid=a, i=b),
//        4 frag_offset(mb=a, r=b, g=c, s=d), 5 pieces per thread, 6 bytes per unit
template <int MB, int GC>
static int fewrow_index(int which, int a, int b, int c, int d) {
    typedef FewRowStageMap<MB, GC, 512> M;
    switch (which) {
        case 0: return M::piece_unit(a, b);
        case 1: return M::piece_row(a, b);
        case 2: return M::piece_index(a);
        case 3: return M::piece_dst(a, b);
        case 4: return M::frag_offset(a, b, c, d);
        case 5: return M::XP;
        case 6: return M::CHUNK_BYTES;
    }
    return -1;
}
extern "C" {


int kernl_idx_rowperm16(int i) { return rowperm16(i); }

int kernl_idx_swz_offset(int row_bytes, int row, int chunk) {
    if (row_bytes == 64) return swz_offset<64>(row, chunk);
    if (row_bytes == 128) return swz_offset<128>(row, chunk);
    if (row_bytes == 256) return swz_offset<256>(row, chunk);
    return -1;
}

// which: 0 stage_row(qd), 1 k_stage_chunk(qd), 2 v_stage_chunk(qd), 3 k_frag_offset(lr=a, lh=b, ks=c),
//        4 v_frag_offset(lane=a, d=b); head size 64 or 128
int kernl_idx_attention(int head_size, int which, int a, int b, int c) {
    if (head_size == 64) {
        typedef AttnTileMap<64> M;
        switch (which) {
            case 0: return M::stage_row(a);
            case 1: return M::k_stage_chunk(a);
            case 2: return M::v_stage_chunk(a);
            case 3: return M::k_frag_offset(a, b, c);
            case 4: return M::v_frag_offset(a, b);
        }
    } else if (head_size == 128) {
        typedef AttnTileMap<128> M;
        switch (which) {
            case 0: return M::stage_row(a);
            case 1: return M::k_stage_chunk(a);
            case 2: return M::v_stage_chunk(a);
            case 3: return M::k_frag_offset(a, b, c);
            case 4: return M::v_frag_offset(a, b);
        }
    }
    return -1;
}

// which: 0 stage_row(i=a, lane=b), 1 stage_chunk(i=a, lane=b), 2 read_offset(lr=a, lh=b, j=c); element size 4 or 2
int kernl_idx_mask(int element_size, int which, int a, int b, int c) {
    if (element_size == 4) {
        typedef MaskTileMap<4> M;
        switch (which) {
            case 0: return M::stage_row(a, b);
            case 1: return M::stage_chunk(a, b);
            case 2: return M::read_offset(a, b, c);
        }
    } else if (element_size == 2) {
        typedef MaskTileMap<2> M;
        switch (which) {
            case 0: return M::stage_row(a, b);
            case 1: return M::stage_chunk(a, b);
            case 2: return M::read_offset(a, b, c);
        }
    }
    return -1;
}

// layout: 0 = 256 columns, 1 = 192 columns, 2 = gated (256 columns)
int kernl_idx_wide_weight_row(int layout, int row) {
    if (layout == 0) return wide_weight_row<false, 8>(row);
    if (layout == 1) return wide_weight_row<false, 6>(row);
    if (layout == 2) return wide_weight_row<true, 8>(row);
    return -1;
}

int kernl_idx_xcd_contiguous(int b, int n) { return xcd_contiguous_index(b, n); }

// which: 0 load_row(q=a), 1 load_chunk(q=a), 2 frag_offset(row=a, kstep=b, g=c)
int kernl_idx_small_tile(int which, int a, int b, int c) {
    switch (which) {
        case 0: return SmallTileMap::load_row(a);
        case 1: return SmallTileMap::load_chunk(a);
        case 2: return SmallTileMap::frag_offset(a, b, c);
    }
    return -1;
}

int kernl_idx_fewrow(int row_blocks, int units_per_stage, int which, int a, int b, int c, int d) {
    if (row_blocks == 1 && units_per_stage == 4) return fewrow_index<1, 4>(which, a, b, c, d);
    if (row_blocks == 2 && units_per_stage == 2) return fewrow_index<2, 2>(which, a, b, c, d);
    if (row_blocks == 4 && units_per_stage == 2) return fewrow_index<4, 2>(which, a, b, c, d);
    if (row_blocks == 8 && units_per_stage == 2) return fewrow_index<8, 2>(which, a, b, c, d);
    return -1;
}

}  // extern "C"
