// Index arithmetic of the kernels whose addressing is easy to get wrong, as plain functions that compile for the
// device and for the host: the kernels call them, and a host program (tests/cpp/host_index_model_test.cpp) walks
// every block, wavefront, lane and stage of every instantiation through the same functions and checks that each
// LDS and global offset is in bounds, that a stage's bytes land where the fragment reads expect them, and that every
// output element is written exactly once.  (The reference keeps such host models beside its own kernels:
// crates/backend-rocm/src/gemm_model.rs, paged_kv_model.rs, norm_model.rs.)
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#define FA_HD __host__ __device__ __forceinline__ constexpr
#else
#define FA_HD inline constexpr
#endif

namespace fa {
namespace ixm {

// ------------------------------------------------------------------ large-tile GEMM (gemm_mfma_big_kernel)
// Block tile 256 rows x NTB * 16 columns, NWAVES = 2 WM wavefronts (WM along m, 2 along n).  One stage is 128 bytes
// of k: 16 A tiles and NTB B tiles of 2 KiB, each moved as two 1 KiB slices by direct global -> LDS loads that
// write 16 bytes per lane at slice base + lane * 16.
constexpr int kBigTk = 128, kBigTile = 2048, kBigRows = 256;
constexpr int kBigStagesA = 3, kBigStagesB = 2;

template <int NTB>
struct BigLds {
    static constexpr int a_stage = 16 * kBigTile, b_stage = NTB * kBigTile;
    static constexpr int b_base = kBigStagesA * a_stage;
    static constexpr int bytes = b_base + kBigStagesB * b_stage;
};

// Blocks of one XCD (the hardware deals consecutive ids round-robin over 8 XCDs) take consecutive tiles, m fastest.
// With eight or more row blocks and a whole number of column blocks per XCD, an XCD walks its column blocks for eight
// row blocks at a time: the 32 tiles its compute units hold together are then 8 x 4 (12 operand panels per k step)
// rather than 16 x 2 or 32 x 1 (18 or 33), which is what its L2 has to fetch.
FA_HD void big_block_tile(uint32_t bid, uint32_t m_blocks, uint32_t n_blocks, uint32_t *mb, uint32_t *nb) {
    const uint32_t total = m_blocks * n_blocks;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
    if (n_blocks % 8 == 0 && m_blocks % 8 == 0) {
        const uint32_t nb8 = n_blocks / 8, xcd = bid / (total / 8), l = bid % (total / 8);
        const uint32_t chunk = l / (8 * nb8), r = l % (8 * nb8);
        *mb = chunk * 8 + r % 8;
        *nb = xcd * nb8 + r / 8;
        return;
    }
    *mb = bid % m_blocks;
    *nb = bid / m_blocks;
}

// A tile (of 16 rows) that wavefront `wave` moves with its load pair i, and the tile-local row of lane `lane`.
template <int NWAVES>
FA_HD int big_a_tile(int wave, int i) { return wave + NWAVES * i; }
FA_HD int big_a_row(int lane) { return lane / 4; }
// Byte offset inside the row's 128 stage bytes that lane `lane` fetches with load x (0 or 1) of a pair, r = lane / 4,
// p = lane % 4 its slot in the row's four slots of slice x.  e4m3: the 16-byte piece q = 2 ((p - r / 2) mod 4) + x.
// int8: piece q = 2 j + x sits in slot (x + 2 (j % 2) + j / 2 + r / 2) mod 4, so that the four k-groups g of k-step s
// (pieces 4 s + g: j = 2 s + g / 2, x = g % 2) read slots (g + s + r / 2) mod 4, the e4m3 pattern: the LDS serves a
// 16-byte read sixteen lanes per cycle, lanes of two neighbouring k-groups together, and any other spacing of their
// slots halves its rate (measured: 8 instead of 4 cycles per instruction).
template <bool FP8>
FA_HD int big_a_src_byte(int lane, int x) {
    const int r = lane / 4, p4 = lane % 4;
    if (FP8) return ((p4 - r / 2) & 3) * 32 + x * 16;
    const int t = (p4 - x - r / 2) & 3;              // = 2 (j % 2) + j / 2
    const int j = ((t & 1) << 1) | (t >> 1);
    return j * 32 + x * 16;
}
// LDS byte offset of the slice that load (tile, h) of stage slot `slot` fills (the lane's 16 bytes go to + lane * 16).
template <int NTB>
FA_HD int big_a_lds_slice(int slot, int tile, int h) { return slot * BigLds<NTB>::a_stage + tile * kBigTile + h * 1024; }
// Byte offsets, inside an A tile of a stage, of the two 16-byte operand reads of lane `lane`: e4m3 reads k bytes
// 32 g .. 32 g + 15 (sub 0) and 32 g + 16 .. + 31 (sub 1) of row r; int8 reads k bytes 64 sub + 16 g .. + 15
// (k-step `sub` of the stage), g = lane / 16, r = lane % 16.
template <bool FP8>
FA_HD int big_a_frag_off(int lane, int sub) {
    const int g = lane / 16, r = lane % 16;
    if (FP8) return sub * 1024 + (4 * r + ((g + r / 2) & 3)) * 16;
    return (g & 1) * 1024 + (4 * r + ((g + sub + r / 2) & 3)) * 16;
}

// B tile (block-local column tile) that wavefront `wave` moves with load pair i: a block of 14 tiles has no tiles
// 14, 15, the wavefronts that would move them repeat tiles 0, 1.
template <int NTB, int NWAVES>
FA_HD int big_b_tile(int wave, int i) { return (wave + NWAVES * i) % NTB; }
// Byte offset, inside the 2 KiB weight tile of a stage in memory, of lane `lane`'s 16 bytes of slice h: e4m3 tiles
// hold 32 bytes per lane (slice h = its half h), int8 stages are two adjacent 1 KiB tiles of 16 bytes per lane.
template <bool FP8>
FA_HD int big_b_src_byte(int lane, int h) { return FP8 ? lane * 32 + h * 16 : h * 1024 + lane * 16; }
template <int NTB>
FA_HD int big_b_lds_slice(int slot, int tile, int h) {
    return BigLds<NTB>::b_base + slot * BigLds<NTB>::b_stage + tile * kBigTile + h * 1024;
}
// First byte, inside a stage's B region, of the fragment (tile j of wavefront column wn, slice h) of lane `lane`.
template <int NTB>
FA_HD int big_b_frag_off(int wn, int j, int h, int lane) { return (wn * (NTB / 2) + j) * kBigTile + h * 1024 + lane * 16; }

// SwiGLU form of the large-tile kernel (weight = gate columns, then up columns, f_tiles column tiles each): the block
// of column index nb owns NTB / 2 tiles of the product; block-local tile `local` = wn * (NTB / 2) + j of wavefront
// column wn is, for j < NTB / 4, gate tile nb * NTB / 2 + wn * NTB / 4 + j, and for j >= NTB / 4 the up tile of the
// same product tile as j - NTB / 4: gate and up of an element sit in the same lane of accumulator tiles j and
// j + NTB / 4.
template <int NTB>
FA_HD uint32_t big_swiglu_tile(uint32_t nb, int local, uint32_t f_tiles) {
    const int wn = local / (NTB / 2), j = local % (NTB / 2);
    const uint32_t prod_tile = nb * (NTB / 2) + wn * (NTB / 4) + j % (NTB / 4);
    return (j < NTB / 4 ? 0 : f_tiles) + prod_tile;
}

// Output element e (0 .. 3) of accumulator tile (i, j) of wavefront (wm, wn) in lane `lane`, block-local: the matrix
// instructions take the weight fragment first, so a lane holds row lane % 16 and columns 4 (lane / 16) + e.
template <int NTB, int WM>
FA_HD void big_out_elem(int wm, int wn, int i, int j, int e, int lane, int *row, int *col) {
    *row = (wm * (16 / WM) + i) * 16 + lane % 16;
    *col = (wn * (NTB / 2) + j) * 16 + 4 * (lane / 16) + e;
}

// ------------------------------------------------------------------ streamed paged attention (decode_stream_kernel)
// The pages of all sequences, laid end to end, are cut into ranges of `per` pages; range r owns pages
// [r per, (r + 1) per) of that axis and leaves one partial result per sequence it touches, in slot r + b.
FA_HD uint32_t stream_range_pages(uint32_t total_pages, uint32_t n_ranges, uint32_t min_pages) {
    const uint32_t per = (total_pages + n_ranges - 1) / n_ranges;
    return per < min_pages ? min_pages : per;
}
// Pages [lo, hi) of a sequence (in its own numbering) that range [rlo, rhi) covers; the sequence occupies [sb, eb)
// of the axis and overlaps the range.
FA_HD void stream_segment(uint32_t rlo, uint32_t rhi, uint32_t sb, uint32_t eb, uint32_t *lo, uint32_t *hi) {
    *lo = (rlo > sb ? rlo : sb) - sb;
    *hi = (rhi < eb ? rhi : eb) - sb;
}
FA_HD uint32_t stream_slot(uint32_t r, uint32_t b) { return r + b; }
// Ranges whose partial results the merge of a sequence adds: the sequence starts at page `pre` of the axis and
// holds npg pages.  An empty sequence has none (lo > hi).
FA_HD void stream_merge_ranges(uint32_t pre, uint32_t npg, uint32_t per, uint32_t *r_lo, uint32_t *r_hi) {
    *r_lo = npg ? pre / per : 1;
    *r_hi = npg ? (pre + npg - 1) / per : 0;
}

// ------------------------------------------------------------------ split-k decode linears (w8a8 / w8a16_ksplit_kernel)
// Block `bid` of a launch with S members per group: the members of a group are S blocks that differ by multiples
// of 8 (one XCD).  A launch has 8 S ceil(n_groups / 8) blocks; groups at or past n_groups return at once.
FA_HD void ksplit_block(uint32_t bid, uint32_t s, uint32_t *group, uint32_t *member) {
    const uint32_t xcd = bid % 8, q = bid / 8;
    *group = (q / s) * 8 + xcd;
    *member = q % s;
}
FA_HD void ksplit_k_range(uint32_t k_tiles, uint32_t member, uint32_t s, uint32_t *lo, uint32_t *hi) {
    *lo = (uint32_t)((uint64_t)k_tiles * member / s);
    *hi = (uint32_t)((uint64_t)k_tiles * (member + 1) / s);
}
// First element of the partial tile set of (group, member) in the workspace; nacc = row tiles x S x 4 items of 64 lanes.
FA_HD uint64_t ksplit_partial_base(uint32_t group, uint32_t member, uint32_t s, uint32_t nacc) {
    return ((uint64_t)group * s + member) * ((uint64_t)nacc * 64);
}
// Activation operand of the decode-shape int8 kernels (w8a8_skinny_kernel, w8a8_ksplit_kernel): byte offset of the 16
// bytes lane `lane` fetches for row tile i and k-tile kt from the tiled codes of m rows (ceil(m / 16) row tiles of
// k_tiles x 1 KiB; lane l holds row l % 16, k-group l / 16).  The lanes of rows at or past m fetch row 0 of their
// k-group instead, and a row tile that lies wholly at or past m (a kernel built for four row tiles under 33 to 48
// rows) is fetched from row tile 0: the buffer holds no such tile.  What they fetch only reaches accumulator rows
// that are never stored.
FA_HD uint32_t decode_a_tile(uint32_t i, uint32_t m) { return i * 16 < m ? i : 0u; }          // the same in every lane
FA_HD uint32_t decode_a_lane_byte(uint32_t i, uint32_t lane, uint32_t m) { return (i * 16 + lane % 16 < m ? lane : lane & 48u) * 16; }
FA_HD uint64_t decode_a_byte(uint32_t i, uint32_t kt, uint32_t lane, uint32_t m, uint32_t k_tiles) {
    return ((uint64_t)decode_a_tile(i, m) * k_tiles + kt) * 1024 + decode_a_lane_byte(i, lane, m);
}
// The weight-stationary split-k linear (w8a8_wstat_ksplit_kernel) leaves a partial tile set per row group: first
// element of the set of (group, member, row group) in its workspace; nacc = row tiles of a row group x S x 4 items.
FA_HD uint64_t rows_ksplit_partial_base(uint32_t group, uint32_t member, uint32_t s, uint32_t row_groups, uint32_t row_group,
                                        uint32_t nacc) {
    return (((uint64_t)group * s + member) * row_groups + row_group) * ((uint64_t)nacc * 64);
}

}  // namespace ixm
}  // namespace fa
