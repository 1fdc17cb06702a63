// Index arithmetic of the kernels' LDS layouts, kept apart from everything that needs a GPU: the kernels include this
// header (through common.h) and so does the host-side replay tool (index_math_host.cpp, built with g++), which walks
// the same functions lane by lane on the CPU.  Nothing in here may depend on HIP types.
#pragma once

#if defined(__HIPCC__)
#define KERNL_HD __host__ __device__ __forceinline__
#else
#define KERNL_HD inline
#endif

namespace kernl {

// Element v (0..15) of lane l of a 32x32 MFMA result is row 8*(v/4) + 4*(l/32) + (v%4), column l % 32.  Feeding MFMA
// row i with logical row rowperm16(i) therefore makes every lane end up with 16 CONSECUTIVE logical rows: lane half h
// holds logical rows 16*h + v for v = 0..15.
KERNL_HD int rowperm16(int i) { return 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3); }

// LDS swizzle for tiles whose rows are ROW_BYTES long (64, 128 or 256) and are read as 16-byte chunks by the
// 32 rows x 2 k-halves pattern of an MFMA operand fetch: 16 consecutive rows reading the same logical chunk
// land in 16 different 16-byte bank groups.
template <int ROW_BYTES>
KERNL_HD int swz_chunk(int row, int chunk) {
    static_assert(ROW_BYTES == 64 || ROW_BYTES == 128 || ROW_BYTES == 256, "row must span 4, 8 or 16 chunks");
    if (ROW_BYTES == 64) return chunk ^ ((row >> 2) & 3);
    if (ROW_BYTES == 128) return chunk ^ ((row >> 1) & 7);
    return chunk ^ (row & 15);
}
template <int ROW_BYTES>
KERNL_HD int swz_offset(int row, int chunk) {  // byte offset inside the tile
    return row * ROW_BYTES + swz_chunk<ROW_BYTES>(row, chunk) * 16;
}

// ----------------------------------------------------------------------------------------------------
// Streaming attention kernel: one stage holds a K tile [64 keys][D] and a V tile [64 keys][D] of 16-bit values,
// row-major, K at byte 0 and V at byte K_BYTES of the stage.
//   staging   the 16-byte chunk at LDS position qd (byte 16 qd of its tile; thread tid owns qd = tid + 256 i) is
//             filled with chunk `k_stage_chunk(qd)` of K row `stage_row(qd)`, resp. `v_stage_chunk(qd)` of the V row
//   K reads   lane (lr = lane % 32, lh = lane / 32) reads, for 32-key block nb and k-step ks, the 16 bytes at
//             nb * 32 * KROW + k_frag_offset(lr, lh, ks): features 16 ks + 8 lh .. +7 of key 32 nb + lr
//   V reads   transposing 8-byte reads (in every group of 16 lanes, lane i hands in the address of 4 consecutive
//             features of one key and receives 4 consecutive keys of feature column i of the 4-key x 16-feature block
//             the group's addresses describe); for 16-key slab ps and 32-feature block d the lane reads at
//             K_BYTES + 16 ps * VP + v_frag_offset(lane, d) and again 8 rows (keys) further down
// ----------------------------------------------------------------------------------------------------
template <int D>
struct AttnTileMap {
    static constexpr int BN = 64, KROW = D * 2, VP = D * 2, K_BYTES = BN * KROW, V_BYTES = BN * VP;
    static constexpr int DC = D / 8, KI = BN * DC / 256;
    static KERNL_HD int stage_row(int qd) { return qd / DC; }
    static KERNL_HD int k_stage_chunk(int qd) { return swz_chunk<KROW>(qd / DC, qd % DC); }
    static KERNL_HD int v_stage_chunk(int qd) {
        const int row = qd / DC, cs = qd % DC;
        const int vsw = (D == 64) ? ((row >> 1) & 1) : (row & 3);
        return cs ^ (vsw << 2);
    }
    static KERNL_HD int k_frag_offset(int lr, int lh, int ks) { return swz_offset<KROW>(lr, 2 * ks + lh); }
    static KERNL_HD int v_frag_offset(int lane, int d) {
        const int i16 = lane & 15, g16 = lane >> 4, lh = lane >> 5;
        const int kq = i16 >> 2;                                    // key of the 4-key group this lane addresses
        const int fs = rowperm16(16 * (g16 & 1) + 4 * (i16 & 3));   // first of its 4 consecutive features
        const int vsw = (D == 64) ? (kq >> 1) : kq;
        return (4 * lh + kq) * VP + ((d ^ vsw) * 64) + fs * 2;
    }
};

// ----------------------------------------------------------------------------------------------------
// Matrix masks of the streaming attention kernel (head size 64): every wave keeps the 32 query rows x 64 keys it needs
// of the current key tile in an LDS region of its own, row r at byte r * ROW with its 16-byte chunks XOR-swizzled.
//   staging   load i of lane `lane` writes the 16 bytes at LDS byte 1024 i + 16 lane and fetches chunk
//             `stage_chunk(i, lane)` of mask row `stage_row(i, lane)` (4 fp32 rows or 8 16-bit rows per load)
//   reads     lane (lr, lh) needs, for j = 0..7, the 4 keys 8 j + 4 lh .. +3 of its row lr: 16 bytes at
//             read_offset(lr, lh, j) for fp32, 8 bytes for 16-bit values
// ----------------------------------------------------------------------------------------------------
template <int ESIZE>
struct MaskTileMap {
    static_assert(ESIZE == 4 || ESIZE == 2, "fp32 or 16-bit mask values");
    static constexpr int ROW = 64 * ESIZE, LOADS = 32 * ROW / 1024;
    static KERNL_HD int stage_row(int i, int lane) { return ESIZE == 4 ? i * 4 + (lane >> 4) : i * 8 + (lane >> 3); }
    static KERNL_HD int stage_chunk(int i, int lane) {
        const int r = stage_row(i, lane);
        return ESIZE == 4 ? ((lane & 15) ^ (r & 15)) : ((lane & 7) ^ ((r >> 1) & 7));
    }
    static KERNL_HD int read_offset(int lr, int lh, int j) {
        if (ESIZE == 4) return lr * ROW + (((2 * j + lh) ^ (lr & 15)) << 4);
        return lr * ROW + ((j ^ ((lr >> 1) & 7)) << 4) + lh * 8;
    }
};

// ----------------------------------------------------------------------------------------------------
// Wide linear kernels: which weight row (inside the tile) LDS row `row` of the weight tile carries.  LDS row `row` is
// row r = row % 16 of 16-row block j of a wave's weight rows (128 per wave in 256-column tiles, 96 in 192-column tiles),
// and lane l16 of the wave receives the results of row r = l16 of every block.  The placement gives that lane
// consecutive output columns:
//   plain    block j row r carries weight row NBN r + j of the wave's rows: lane l16 holds columns NBN l16 .. + NBN - 1
//   gated    the fused weight holds 32 gate rows, then the 32 value rows of the same 32 output columns, and so on; blocks
//            0 .. 3 carry the gate rows and blocks 4 .. 7 the value rows of output columns c = 4 r + j % 4 (of the wave's
//            64): fused row 64 (c / 32) + 32 (j / 4) + c % 32
// ----------------------------------------------------------------------------------------------------
template <bool GATED, int NBN>
KERNL_HD int wide_weight_row(int row) {
    const int r = row & 15;
    if (GATED) {
        const int j = (row >> 4) & 7, c = 4 * r + (j & 3);
        return (row & ~127) + 64 * (c >> 5) + 32 * (j >> 2) + (c & 31);
    }
    const int per_wave = 16 * NBN, first = (row / per_wave) * per_wave;
    return first + NBN * r + ((row - first) >> 4);
}

// ----------------------------------------------------------------------------------------------------
// Stream-K few-row linear kernel: a stage of x holds GC units (64-wide chunks of K), unit j at byte j * CHUNK_BYTES, as
// MP = 16 MB rows of 128 bytes whose eight 16-byte pieces are XOR-swizzled.
//   staging   piece i of thread tid is 16-byte piece piece_index(tid) of row piece_row(tid, i) of the group's unit
//             piece_unit(tid, i) (q = tid + THREADS i walks unit, row, piece), stored at piece_dst(tid, i)
//   reads     lane (r = lane % 16, g = lane / 16) takes, for 16-row block mb and k-step s, the 16 bytes at
//             frag_offset(mb, r, g, s) of the unit: k = 16 g + 8 s .. + 7 of x row 16 mb + r
// ----------------------------------------------------------------------------------------------------
template <int MB, int GC, int THREADS>
struct FewRowStageMap {
    static constexpr int MP = 16 * MB, CHUNK_BYTES = MP * 128, XP = GC * MP * 8 / THREADS;
    static_assert(GC * MP * 8 % THREADS == 0 && XP >= 1, "every thread stages the same number of pieces");
    static KERNL_HD int piece_unit(int tid, int i) { return (tid + THREADS * i) / (MP * 8); }
    static KERNL_HD int piece_row(int tid, int i) { return ((tid + THREADS * i) >> 3) % MP; }
    static KERNL_HD int piece_index(int tid) { return tid & 7; }
    static KERNL_HD int piece_dst(int tid, int i) {
        return piece_unit(tid, i) * CHUNK_BYTES + swz_offset<128>(piece_row(tid, i), piece_index(tid));
    }
    static KERNL_HD int frag_offset(int mb, int r, int g, int s) { return swz_offset<128>(16 * mb + r, 2 * g + s); }
};

// ----------------------------------------------------------------------------------------------------
// Small-problem linear kernels (linear_small.hip): an operand tile of a k-tile is ROWS rows of 128 bytes (64 k-values)
// whose eight 16-byte chunks are XOR-swizzled.  Tile loads write LDS directly, a wave's load filling 1 KB of consecutive
// LDS: the lane that writes LDS chunk q (byte 16 q of the tile) fetches from memory what belongs there.
//   loads     LDS chunk q holds chunk load_chunk(q) (k = 8 load_chunk(q) .. + 7) of tile row load_row(q)
//   reads     lane (r = lane % 16, g = lane / 16) takes, for 16-row block b and k-step s, the 16 bytes at
//             frag_offset(16 b + r, s, g): k = 32 s + 8 g .. + 7 of that row
// ----------------------------------------------------------------------------------------------------
// Workgroups of a launch are dealt to the 8 XCDs in turn (workgroup b runs on XCD b % 8), and each XCD has an L2 of its
// own.  This maps workgroup b of n to a tile index such that every XCD works on ONE contiguous run of indices: with the
// row tile running fastest in the index, the workgroups that share a weight tile then sit on one XCD at the same time
// and all but the first of them find it in that L2.  A bijection of 0 .. n-1 for every n.
KERNL_HD int xcd_contiguous_index(int b, int n) {
    const int xcd = b % 8, slot = b / 8, base = n / 8, rem = n % 8;
    return xcd * base + (xcd < rem ? xcd : rem) + slot;
}

struct SmallTileMap {
    static constexpr int ROW_BYTES = 128, CHUNKS_PER_ROW = 8;
    static KERNL_HD int load_row(int q) { return q / CHUNKS_PER_ROW; }
    static KERNL_HD int load_chunk(int q) { return swz_chunk<ROW_BYTES>(q / CHUNKS_PER_ROW, q % CHUNKS_PER_ROW); }
    static KERNL_HD int frag_offset(int row, int kstep, int g) { return swz_offset<ROW_BYTES>(row, 4 * kstep + g); }
};

}  // namespace kernl
