// Host model of the kernels' index arithmetic (fandhe_ai_amd/csrc/index_models.hpp: the functions the kernels
// themselves call).  No device: every block, wavefront, lane, load and stage of every instantiation is walked on
// the host and checked for bounds, for agreement between where a stage's bytes are written and where the operand
// reads expect them, and for every output being written exactly once.
//   large-tile GEMM   : e4m3 / int8 x 14 / 16 column tiles x 4 / 8 / 16 wavefronts
//   streamed attention: ranges, segments and partial-result slots against the merge's expectation, ragged lengths
//   split-k linears   : groups on one XCD, k ranges, workspace offsets
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <vector>

#include "../../fandhe_ai_amd/csrc/index_models.hpp"

using namespace fa::ixm;

static int g_checks = 0;
#define CHECK(cond)                                                                      \
    do {                                                                                 \
        ++g_checks;                                                                      \
        if (!(cond)) {                                                                   \
            std::fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                                \
        }                                                                                \
    } while (0)

// ------------------------------------------------------------------ large-tile GEMM
// What an LDS byte of a stage holds: operand row (A: block-local row, B: block-local column) and k byte of the stage.
struct Tag {
    int row = -1, kbyte = -1;
};

template <bool FP8, int NTB, int WM>
static void gemm_case() {
    constexpr int NWAVES = 2 * WM, TPW = 16 / NWAVES, AI = 16 / WM, WNT = NTB / 2;
    using L = BigLds<NTB>;
    static_assert(L::bytes <= 160 * 1024, "stages exceed the LDS of a compute unit");
    // one stage's loads of every wavefront into slot `slot` (A) / `slot % 2` (B)
    for (int slot = 0; slot < kBigStagesA; ++slot) {
        std::vector<Tag> lds(L::bytes);
        std::vector<int> writes(L::bytes, 0);
        for (int wave = 0; wave < NWAVES; ++wave)
            for (int i = 0; i < TPW; ++i)
                for (int h = 0; h < 2; ++h)
                    for (int lane = 0; lane < 64; ++lane) {
                        // A: lane fetches 16 bytes of row (tile * 16 + lane / 4) at big_a_src_byte, lands at slice + lane * 16
                        const int tile = big_a_tile<NWAVES>(wave, i);
                        CHECK(tile >= 0 && tile < 16);
                        const int row = tile * 16 + big_a_row(lane), src = big_a_src_byte<FP8>(lane, h);
                        CHECK(row < kBigRows && src >= 0 && src % 16 == 0 && src + 16 <= kBigTk);
                        const int dst = big_a_lds_slice<NTB>(slot, tile, h) + lane * 16;
                        CHECK(dst >= slot * L::a_stage && dst + 16 <= (slot + 1) * L::a_stage);
                        for (int b = 0; b < 16; ++b) {
                            lds[dst + b] = Tag{row, src + b};
                            writes[dst + b] += 1;
                        }
                        // B: lane's 16 bytes of slice h of the stage's weight tile, lands at slice + lane * 16
                        const int bt = big_b_tile<NTB, NWAVES>(wave, i);
                        CHECK(bt >= 0 && bt < NTB);
                        const int bsrc = big_b_src_byte<FP8>(lane, h);
                        CHECK(bsrc >= 0 && bsrc + 16 <= kBigTile);
                        const int bslot = slot % kBigStagesB;
                        const int bdst = big_b_lds_slice<NTB>(bslot, bt, h) + lane * 16;
                        CHECK(bdst >= L::b_base + bslot * L::b_stage && bdst + 16 <= L::b_base + (bslot + 1) * L::b_stage);
                        for (int b = 0; b < 16; ++b) {
                            // a tile moved twice (14-tile blocks) must bring the same bytes to the same place
                            if (lds[bdst + b].row >= 0) CHECK(lds[bdst + b].row == bt && lds[bdst + b].kbyte == bsrc + b);
                            lds[bdst + b] = Tag{bt, bsrc + b};
                            writes[bdst + b] += 1;
                        }
                    }
        // every byte of the stage's A region exactly once, every byte of its B region at least once
        for (int b = 0; b < L::a_stage; ++b) CHECK(writes[slot * L::a_stage + b] == 1);
        for (int b = 0; b < L::b_stage; ++b) CHECK(writes[L::b_base + (slot % kBigStagesB) * L::b_stage + b] >= 1);
        // every source byte of the stage reaches LDS: 256 rows x 128 bytes of A
        std::set<std::pair<int, int>> seen;
        for (int b = 0; b < L::a_stage; ++b) seen.insert({lds[slot * L::a_stage + b].row, lds[slot * L::a_stage + b].kbyte});
        CHECK((int)seen.size() == kBigRows * kBigTk);

        // operand reads.  A: lane (g, r) of row tile t wants row 16 t + r and, e4m3, k bytes 32 g + 16 sub .. + 15;
        // int8, k bytes 64 sub + 16 g .. + 15.  16-byte reads must also be bank-conflict free.
        for (int wm = 0; wm < WM; ++wm)
            for (int i = 0; i < AI; ++i)
                for (int sub = 0; sub < 2; ++sub) {
                    for (int lane = 0; lane < 64; ++lane) {
                        const int off = slot * L::a_stage + (wm * AI + i) * kBigTile + big_a_frag_off<FP8>(lane, sub);
                        CHECK(off % 16 == 0 && off >= slot * L::a_stage && off + 16 <= (slot + 1) * L::a_stage);
                        const int g = lane / 16, r = lane % 16;
                        const int want_k = FP8 ? 32 * g + 16 * sub : 64 * sub + 16 * g;
                        for (int b = 0; b < 16; ++b) {
                            CHECK(lds[off + b].row == (wm * AI + i) * 16 + r);
                            CHECK(lds[off + b].kbyte == want_k + b);
                        }
                    }
                    for (int oct = 0; oct < 8; ++oct) {      // eight lanes x 16 bytes = all 32 banks once
                        std::set<int> banks;
                        for (int l = 0; l < 8; ++l) banks.insert((big_a_frag_off<FP8>(oct * 8 + l, sub) / 16) % 8);
                        CHECK(banks.size() == 8);
                    }
                    // the full-rate rule as measured on the device: eight lanes of one k-group and the same eight of
                    // the neighbouring group (lanes l and l + 16) are served in one cycle and must cover the 64 banks
                    // (sixteen 16-byte columns) exactly once
                    for (int pair = 0; pair < 2; ++pair)
                        for (int half = 0; half < 2; ++half) {
                            std::set<int> cols;
                            for (int l = 0; l < 8; ++l)
                                for (int gg = 0; gg < 2; ++gg)
                                    cols.insert((big_a_frag_off<FP8>(32 * pair + 16 * gg + 8 * half + l, sub) / 16) % 16);
                            CHECK(cols.size() == 16);
                        }
                }
        // B: lane l of fragment j of wavefront column wn wants slice h of its own 16 bytes of tile wn * WNT + j
        for (int wn = 0; wn < 2; ++wn)
            for (int j = 0; j < WNT; ++j)
                for (int h = 0; h < 2; ++h)
                    for (int lane = 0; lane < 64; ++lane) {
                        const int bslot = slot % kBigStagesB;
                        const int off = L::b_base + bslot * L::b_stage + big_b_frag_off<NTB>(wn, j, h, lane);
                        CHECK(off + 16 <= L::b_base + (bslot + 1) * L::b_stage);
                        for (int b = 0; b < 16; ++b) {
                            CHECK(lds[off + b].row == wn * WNT + j);
                            CHECK(lds[off + b].kbyte == big_b_src_byte<FP8>(lane, h) + b);
                        }
                    }
    }
    // outputs: every element of the 256 x NTB * 16 tile exactly once, four consecutive columns per lane and tile
    std::vector<int> hit(kBigRows * NTB * 16, 0);
    for (int wm = 0; wm < WM; ++wm)
        for (int wn = 0; wn < 2; ++wn)
            for (int i = 0; i < AI; ++i)
                for (int j = 0; j < WNT; ++j)
                    for (int lane = 0; lane < 64; ++lane) {
                        int row0, col0;
                        big_out_elem<NTB, WM>(wm, wn, i, j, 0, lane, &row0, &col0);
                        CHECK(col0 % 4 == 0);                  // the 8 / 16-byte store is aligned
                        for (int e = 0; e < 4; ++e) {
                            int row, col;
                            big_out_elem<NTB, WM>(wm, wn, i, j, e, lane, &row, &col);
                            CHECK(row == row0 && col == col0 + e);
                            CHECK(row >= 0 && row < kBigRows && col >= 0 && col < NTB * 16);
                            hit[row * NTB * 16 + col] += 1;
                        }
                    }
    for (int v : hit) CHECK(v == 1);
}

static void gemm_block_map() {
    for (uint32_t mbs : {1u, 2u, 3u, 8u, 9u, 16u, 32u})
        for (uint32_t nbs : {1u, 4u, 7u, 16u, 24u, 56u, 64u, 112u}) {
            std::set<std::pair<uint32_t, uint32_t>> tiles;
            for (uint32_t bid = 0; bid < mbs * nbs; ++bid) {
                uint32_t mb, nb;
                big_block_tile(bid, mbs, nbs, &mb, &nb);
                CHECK(mb < mbs && nb < nbs);
                tiles.insert({mb, nb});
            }
            CHECK(tiles.size() == (size_t)mbs * nbs);          // a bijection: every tile has one block
        }
    // blocks that the hardware puts on one XCD (same id mod 8) are consecutive tiles
    uint32_t mb0, nb0, mb1, nb1;
    big_block_tile(0, 8, 64, &mb0, &nb0);
    big_block_tile(8, 8, 64, &mb1, &nb1);
    CHECK(nb0 == nb1 && mb1 == mb0 + 1);
}

// ------------------------------------------------------------------ streamed attention
static uint32_t rng_state = 12345;
static uint32_t rnd(uint32_t n) {
    rng_state = rng_state * 1664525u + 1013904223u;
    return (rng_state >> 8) % n;
}

static void stream_case(const std::vector<uint32_t> &pages, uint32_t n_ranges, uint32_t min_pages) {
    const uint32_t batch = (uint32_t)pages.size();
    uint32_t total = 0;
    for (uint32_t p : pages) total += p;
    const uint32_t per = stream_range_pages(total, n_ranges, min_pages);
    CHECK(per >= 1 || total == 0);
    // what the streaming kernel writes: slot -> (sequence, covered pages)
    std::map<uint32_t, std::pair<uint32_t, uint32_t>> slots;
    std::vector<std::vector<int>> covered(batch);
    for (uint32_t b = 0; b < batch; ++b) covered[b].assign(pages[b], 0);
    std::vector<std::set<uint32_t>> ranges_of(batch);
    for (uint32_t r = 0; r < n_ranges; ++r) {
        const uint64_t rlo64 = (uint64_t)r * per;
        if (rlo64 >= total) continue;
        const uint32_t rlo = (uint32_t)rlo64, rhi = rlo + per < total ? rlo + per : total;
        uint32_t base = 0;
        for (uint32_t b = 0; b < batch; ++b) {
            const uint32_t sb = base, eb = base + pages[b];
            base = eb;
            if (!(pages[b] != 0 && sb < rhi && eb > rlo)) continue;
            uint32_t lo, hi;
            stream_segment(rlo, rhi, sb, eb, &lo, &hi);
            CHECK(lo < hi && hi <= pages[b]);
            for (uint32_t pg = lo; pg < hi; ++pg) covered[b][pg] += 1;
            const uint32_t slot = stream_slot(r, b);
            CHECK(slot < n_ranges + batch);                    // the workspace holds n_ranges + batch slots
            CHECK(slots.find(slot) == slots.end());            // no two partial results share a slot
            slots[slot] = {b, hi - lo};
            ranges_of[b].insert(r);
        }
    }
    // every page of every sequence streamed exactly once; the merge reads exactly the slots that were written
    uint32_t pre = 0;
    for (uint32_t b = 0; b < batch; ++b) {
        for (int c : covered[b]) CHECK(c == 1);
        uint32_t r_lo, r_hi;
        stream_merge_ranges(pre, pages[b], per, &r_lo, &r_hi);
        std::set<uint32_t> want;
        for (uint32_t r = r_lo; r <= r_hi && r_lo <= r_hi; ++r) want.insert(r);
        CHECK(want == ranges_of[b]);
        for (uint32_t r : want) CHECK(slots.at(stream_slot(r, b)).first == b);
        pre += pages[b];
    }
}

static void stream_cases() {
    stream_case({1}, 128, 1);
    stream_case({0, 0, 3}, 4, 1);
    stream_case({5, 0, 7, 1}, 3, 2);
    stream_case({64, 512, 8, 300}, 128, 4);
    for (int t = 0; t < 300; ++t) {
        const uint32_t batch = 1 + rnd(64);
        std::vector<uint32_t> pages(batch);
        for (auto &p : pages) p = rnd(4) == 0 ? 0 : rnd(600);
        stream_case(pages, 1 + rnd(300), 1 + rnd(8));
    }
}

// ------------------------------------------------------------------ split-k linears
static void ksplit_cases() {
    for (uint32_t s : {2u, 4u})
        for (uint32_t n_groups : {1u, 7u, 8u, 64u, 65u, 688u})
            for (uint32_t k_tiles : {32u, 64u, 65u, 172u, 224u})
                for (uint32_t mt : {1u, 2u}) {
                    const uint32_t blocks = 8 * s * ((n_groups + 7) / 8), nacc = mt * s * 4;
                    std::map<uint32_t, std::set<uint32_t>> members, xcds;
                    for (uint32_t bid = 0; bid < blocks; ++bid) {
                        uint32_t group, member;
                        ksplit_block(bid, s, &group, &member);
                        CHECK(member < s);
                        CHECK(members[group].insert(member).second);       // every (group, member) once
                        xcds[group].insert(bid % 8);
                    }
                    for (uint32_t g = 0; g < n_groups; ++g) {
                        CHECK(members[g].size() == s);                     // whole groups only
                        CHECK(xcds[g].size() == 1);                        // on one XCD
                        uint32_t next = 0;
                        for (uint32_t m = 0; m < s; ++m) {
                            uint32_t lo, hi;
                            ksplit_k_range(k_tiles, m, s, &lo, &hi);
                            CHECK(lo == next && hi >= lo);                 // the members' k ranges tile [0, k_tiles)
                            next = hi;
                            const uint64_t base = ksplit_partial_base(g, m, s, nacc);
                            CHECK(base + (uint64_t)nacc * 64 <= (uint64_t)n_groups * s * nacc * 64);
                            CHECK(base % ((uint64_t)nacc * 64) == 0);
                        }
                        CHECK(next == k_tiles);
                    }
                }
}

// The weight-stationary split-k linear: partial tile sets of (group, member, row group) tile its workspace without
// gaps or overlaps, and the k-tiles of a member's eight wavefronts (step t of wavefront w: lo + w + 8 t) cover the
// member's range exactly once within the kernel's register depth.
static void rows_ksplit_cases() {
    const uint32_t s = 4, nacc = 2 * s * 4;
    for (uint32_t n_groups : {1u, 8u, 64u, 65u})
        for (uint32_t row_groups : {3u, 10u, 16u}) {
            std::set<uint64_t> bases;
            const uint64_t total = (uint64_t)n_groups * s * row_groups * nacc * 64;
            for (uint32_t g = 0; g < n_groups; ++g)
                for (uint32_t m = 0; m < s; ++m)
                    for (uint32_t rg = 0; rg < row_groups; ++rg) {
                        const uint64_t base = rows_ksplit_partial_base(g, m, s, row_groups, rg, nacc);
                        CHECK(base % ((uint64_t)nacc * 64) == 0 && base + (uint64_t)nacc * 64 <= total);
                        CHECK(bases.insert(base).second);
                    }
            CHECK(bases.size() * nacc * 64 == total);
        }
    for (uint32_t k_tiles : {128u, 160u, 172u, 224u}) {
        const uint32_t per_wave = ((k_tiles + 3) / 4 + 7) / 8, ktw = per_wave <= 4 ? 4 : 7;
        for (uint32_t m = 0; m < s; ++m) {
            uint32_t lo, hi;
            ksplit_k_range(k_tiles, m, s, &lo, &hi);
            std::set<uint32_t> seen;
            for (uint32_t w = 0; w < 8; ++w) {
                const uint32_t len = hi - lo, cnt = len > w ? (len - w + 7) / 8 : 0;
                CHECK(cnt <= ktw);
                for (uint32_t t = 0; t < cnt; ++t) CHECK(seen.insert(lo + w + 8 * t).second);
            }
            CHECK(seen.size() == hi - lo && (seen.empty() || (*seen.begin() == lo && *seen.rbegin() == hi - 1)));
        }
    }
}

// Activation fetch of the decode-shape int8 kernels: for every row count the kernels take, under the exact number of
// row tiles (w8a8_skinny_kernel) and under the 1 / 2 / 4 the split-k form is built in (four row tiles from 33 rows on),
// every lane's 16 bytes lie inside the tiled codes of ceil(m / 16) row tiles, a lane of a row below m fetches its own
// row and k-group, and every other lane fetches bytes that some lane of a row below m fetches too.
static void decode_a_cases() {
    for (uint32_t k_tiles : {1u, 2u, 65u, 224u})
        for (uint32_t m = 1; m <= 64; ++m) {
            const uint32_t tiles = (m + 15) / 16;
            const uint64_t bytes = (uint64_t)tiles * k_tiles * 1024;
            for (uint32_t mt : {tiles, m <= 16 ? 1u : m <= 32 ? 2u : 4u})
                for (uint32_t kt : {0u, k_tiles / 2, k_tiles - 1}) {
                    std::set<uint64_t> own;
                    for (uint32_t i = 0; i < mt; ++i)
                        for (uint32_t lane = 0; lane < 64; ++lane) {
                            const uint64_t b = decode_a_byte(i, kt, lane, m, k_tiles);
                            CHECK(b % 16 == 0 && b + 16 <= bytes);
                            if (i * 16 + lane % 16 < m) {
                                CHECK(b == ((uint64_t)i * k_tiles + kt) * 1024 + lane * 16);
                                own.insert(b);
                            }
                        }
                    for (uint32_t i = 0; i < mt; ++i)
                        for (uint32_t lane = 0; lane < 64; ++lane) CHECK(own.count(decode_a_byte(i, kt, lane, m, k_tiles)) == 1);
                }
        }
}

// SwiGLU form of the large-tile kernel: over all blocks every gate tile and every up tile of the weight is taken exactly
// once, and accumulator tiles j and j + NTB / 4 of a wavefront column are gate and up of the same product tile.
template <int NTB>
static void swiglu_tile_case(uint32_t f_tiles) {
    std::set<uint32_t> seen;
    const uint32_t n_blocks = f_tiles / (NTB / 2);
    for (uint32_t nb = 0; nb < n_blocks; ++nb)
        for (int wn = 0; wn < 2; ++wn)
            for (int j = 0; j < NTB / 4; ++j) {
                const uint32_t g = big_swiglu_tile<NTB>(nb, wn * (NTB / 2) + j, f_tiles);
                const uint32_t u = big_swiglu_tile<NTB>(nb, wn * (NTB / 2) + j + NTB / 4, f_tiles);
                CHECK(g < f_tiles && u == g + f_tiles);
                CHECK(g == nb * (NTB / 2) + wn * (NTB / 4) + j);           // the product tile the epilogue writes
                CHECK(seen.insert(g).second && seen.insert(u).second);
            }
    CHECK(seen.size() == 2 * (size_t)f_tiles);
}

int main() {
    swiglu_tile_case<16>(8);
    swiglu_tile_case<16>(896);
    swiglu_tile_case<8>(8);
    swiglu_tile_case<8>(896);
    rows_ksplit_cases();
    decode_a_cases();
    gemm_case<true, 14, 4>();
    gemm_case<true, 16, 4>();
    gemm_case<false, 14, 4>();
    gemm_case<false, 16, 4>();
    gemm_case<false, 8, 4>();
    gemm_case<true, 14, 2>();
    gemm_case<true, 16, 2>();
    gemm_case<false, 14, 2>();
    gemm_case<false, 16, 2>();
    gemm_case<true, 14, 8>();
    gemm_case<true, 16, 8>();
    gemm_case<false, 14, 8>();
    gemm_case<false, 16, 8>();
    gemm_block_map();
    stream_cases();
    ksplit_cases();
    std::printf("%d checks ok\n", g_checks);
    return 0;
}
