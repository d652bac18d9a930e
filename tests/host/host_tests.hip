// Host-only checks of the type layer (no GPU needed): layouts, iterators, shapes, the LDS
// swizzle and the workgroup -> tile map. Restates the reference's host-side unit tests
//   tests/cpp/cell/test_layout.cu:105-131 and tests/cpp/cell/test_global_tile_iterator.cu:35-154
// and adds the checks the new LDS layouts need. Exit code = number of failed checks.
#include "kernels/gemm_pipelined.hpp"
#include "types/mod.hpp"

#include <cstdio>
#include <set>
#include <sstream>
#include <vector>

using namespace tiledcuda;
using namespace tiledcuda::cell;
namespace tl = tiledcuda::cell::tile_layout;

static int g_failed = 0;
#define CHECK(...)                                                         \
    do {                                                                   \
        if (!(__VA_ARGS__)) {                                                   \
            ++g_failed;                                                    \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #__VA_ARGS__);  \
        }                                                                  \
    } while (0)

static void test_layout() {
    using Layout1 = tl::RowMajor<4, 7>;
    CHECK(tl::num_rows<Layout1> == 4);
    CHECK(tl::num_cols<Layout1> == 7);
    CHECK(tl::get_numel<Layout1> == 28);
    CHECK(tl::row_stride<Layout1> == 7);
    CHECK(tl::col_stride<Layout1> == 1);
    CHECK(tl::layout_type<Layout1> == tl::Layout::kRowMajor);
    CHECK(std::string(tl::layout_type_to_str(tl::layout_type<Layout1>)) == "RowMajor");

    using Layout2 = tl::ColMajor<4, 7>;
    CHECK(tl::num_rows<Layout2> == 4);
    CHECK(tl::num_cols<Layout2> == 7);
    CHECK(tl::get_numel<Layout2> == 28);
    CHECK(tl::row_stride<Layout2> == 1);
    CHECK(tl::col_stride<Layout2> == 4);
    CHECK(tl::layout_type<Layout2> == tl::Layout::kColMajor);
    CHECK(std::string(tl::layout_type_to_str(tl::layout_type<Layout2>)) == "ColMajor");

    Layout1 l1;
    Layout2 l2;
    CHECK(l1(2, 3) == 17);
    CHECK(l2(2, 3) == 14);
    using Strided = tl::RowMajor<4, 7, 32>;
    CHECK(Strided{}(2, 3) == 67);
    // the documented quirk: a 1x1 column-major layout reads as row-major
    CHECK((tl::layout_type<tl::ColMajor<1, 1>> == tl::Layout::kRowMajor));
}

template <bool kRowMajor>
static void test_gtile_iterator() {
    constexpr int kRows = 4, kCols = 9, kS0 = 2, kS1 = 3;
    using Layout = std::conditional_t<kRowMajor, tl::RowMajor<kRows, kCols>, tl::ColMajor<kRows, kCols>>;
    using Tile = GlobalTile<float, Layout>;
    using Iterator = GTileIterator<Tile, TileShape<kS0, kS1>>;

    std::vector<float> data(kRows * kCols);
    for (int i = 0; i < kRows * kCols; ++i) data[i] = float(i);  // value = memory offset

    CHECK(Iterator::sc0 == kRows / kS0);
    CHECK(Iterator::sc1 == kCols / kS1);

    Iterator iter(data.data());
    for (int i = 0; i < Iterator::sc0; ++i) {
        for (int j = 0; j < Iterator::sc1; ++j) {
            auto tile = iter(i, j);
            for (int m = 0; m < kS0; ++m)
                for (int n = 0; n < kS1; ++n) {
                    const int row = i * kS0 + m, col = j * kS1 + n;
                    const int want = kRowMajor ? row * kCols + col : row + col * kRows;
                    CHECK(int(tile(m, n)) == want);
                }
        }
    }
    // slices: a row strip then a 1-D index along it equals the 2-D index
    for (int i = 0; i < Iterator::sc0; ++i) {
        auto strip = iter(i, _);
        for (int j = 0; j < Iterator::sc1; ++j) CHECK(strip(j).data() == iter(i, j).data());
    }
    for (int j = 0; j < Iterator::sc1; ++j) {
        auto strip = iter(_, j);
        for (int i = 0; i < Iterator::sc0; ++i) CHECK(strip(i).data() == iter(i, j).data());
    }
    CHECK(iter.to_tile().data() == data.data());

    // a sub-tile of a strided parent keeps the parent's strides
    using Big = GlobalTile<float, tl::RowMajor<64, 256, 4096>>;
    using BigIter = GTileIterator<Big, TileShape<64, 32>>;
    BigIter big((float*)nullptr);
    CHECK(BigIter::sc0 == 1 && BigIter::sc1 == 8);
    CHECK(big(3).data() == (float*)nullptr + 96);
    CHECK(decltype(big(3))::kRowStride == 4096);

    std::ostringstream os;
    os << iter;
    CHECK(os.str() == "numel = 36, ChunkShape[2, 3], sc0 = 2, sc1 = 3");
}

static void test_tile_shape_and_regtile() {
    using S = TileShape<4, 5, 6>;
    CHECK(dim_size<0, S> == 4 && dim_size<1, S> == 5 && dim_size<2, S> == 6);
    CHECK(get_numel<S> == 120);

    using RegA = RegTile<BaseTileRowMajor<__half>, tl::RowMajor<2, 4>>;
    using RegB = RegTile<BaseTileColMajor<__half>, tl::ColMajor<4, 3>>;
    CHECK(RegA::kType == tl::Layout::kRowMajor);
    CHECK(RegB::kType == tl::Layout::kColMajor);
    CHECK((RegTile<BaseTileColMajor<float>, tl::ColMajor<1, 1>>::kType == tl::Layout::kColMajor));
    CHECK(sizeof(BaseTileRowMajor<__half>) == 8);   // two K-adjacent tiles are 16 contiguous bytes
    CHECK(sizeof(RegA) == 2 * 4 * 8);
    CHECK(sizeof(BaseTileRowMajor<float>) == 16);
    CHECK(traits::BaseTileShape<__half>::kNumelPerThread == 4);
    CHECK(traits::BaseTileShape<__half>::kTileSize == 16);
    RegA a;
    std::ostringstream os;
    os << a;
    CHECK(os.str() == "RowMajor[32, 64]");
    RegB b;
    std::ostringstream os2;
    os2 << b;
    CHECK(os2.str() == "ColMajor[64, 48]");

    // a freshly constructed register tile is zero (the reference zero-fills in the constructor)
    RegTile<BaseTileRowMajor<float>, tl::RowMajor<2, 2>> c;
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 2; ++j)
            for (int e = 0; e < 4; ++e) CHECK(c(i, j)(0, e) == 0.f);
    c(1, 1)(0, 2) = 5.f;
    c.clear();
    CHECK(c(1, 1)(0, 2) == 0.f);
}

// The swizzle must be a bijection of every line, keep 4-element chunks whole, keep pairs of
// chunks adjacent for 2-byte elements, and (for power-of-two pitches) make the BaseTile
// access pattern of one wavefront pass bank-conflict free.
template <int kPitch, int kElemBytes>
static void test_swizzle(bool expect_conflict_free) {
    using Swz = tl::LdsSwizzle<kPitch, kElemBytes>;
    for (int line = 0; line < 64; ++line) {
        std::set<int> seen;
        for (int e = 0; e < kPitch; ++e) {
            const int p = Swz::apply(line, e);
            CHECK(p >= 0 && p < kPitch);
            seen.insert(p);
            if (e % 4 == 0)
                for (int t = 1; t < 4; ++t) CHECK(Swz::apply(line, e + t) == p + t);
            if (kElemBytes == 2 && e % 8 == 0) CHECK(Swz::apply(line, e + 4) == p + 4 && p % 8 == 0);
        }
        CHECK(int(seen.size()) == kPitch);
    }
    if (!expect_conflict_free) return;
    // one pass of a 64-bit (f16) access = 32 lanes, of a 128-bit (f32) access = 16 lanes:
    // lanes (r = 0..15, g) read the chunk at column 16 * tile + 4 * g of line line0 + r
    const int lanes_per_pass = kElemBytes == 2 ? 32 : 16;
    const int chunk_bytes = 4 * kElemBytes;
    for (int line0 = 0; line0 < 64; line0 += 16) {
        for (int tile = 0; tile < kPitch / 16; ++tile) {
            for (int pass = 0; pass < 64 / lanes_per_pass; ++pass) {
                std::set<int> banks;
                for (int l = 0; l < lanes_per_pass; ++l) {
                    const int lane = pass * lanes_per_pass + l;
                    const int r = lane % 16, g = lane / 16;
                    const int byte = ((line0 + r) * kPitch + Swz::apply(line0 + r, tile * 16 + 4 * g)) * kElemBytes;
                    for (int b = 0; b < chunk_bytes; b += 4) banks.insert(((byte + b) / 4) % 64);
                }
                CHECK(int(banks.size()) == lanes_per_pass * chunk_bytes / 4);
            }
        }
    }
}

// The swizzle for tiles read with the transposing LDS read: a bijection per line that keeps 32-byte units whole and
// repeats every 4 lines; one pass of ds_read_b64_tr_b16 (32 lanes = two 16-lane groups on adjacent 32-byte units, each
// group fetching 4 consecutive lines x 4 x 8 bytes) must touch 64 distinct banks.
template <int kPitch>
static void test_swizzle_tr() {
    using Swz = tl::LdsSwizzleTr<kPitch, 2>;
    CHECK(Swz::kLinePeriod == 4);
    for (int line = 0; line < 64; ++line) {
        std::set<int> seen;
        for (int e = 0; e < kPitch; ++e) {
            const int p = Swz::apply(line, e);
            CHECK(p >= 0 && p < kPitch);
            seen.insert(p);
            if (e % 16 == 0)
                for (int t = 1; t < 16; ++t) CHECK(Swz::apply(line, e + t) == p + t);
            CHECK(Swz::apply(line + 4, e) == p);
        }
        CHECK(int(seen.size()) == kPitch);
    }
    for (int line0 = 0; line0 < 64; line0 += 4) {
        for (int col0 = 0; col0 < kPitch; col0 += 32) {
            std::set<int> banks;
            for (int lane = 0; lane < 32; ++lane) {
                const int L = lane & 15, grp = lane >> 4;
                const int line = line0 + (L >> 2), col = col0 + 16 * grp + 4 * (L & 3);
                const int byte = (line * kPitch + Swz::apply(line, col)) * 2;
                for (int b = 0; b < 8; b += 4) banks.insert(((byte + b) / 4) % 64);
            }
            CHECK(int(banks.size()) == 64);
        }
    }
}

// The 8-line form (operand tiles 16 wide: the two 16-lane groups of a pass sit on the same 32-byte unit of 8 consecutive
// lines, lane group g four lines below group g - 1): a bijection per line that keeps 32-byte units whole, repeats every 8
// lines, and makes every pass of the read touch 64 distinct banks.
template <int kPitch>
static void test_swizzle_tr8() {
    using Swz = tl::LdsSwizzleTr<kPitch, 2, 8>;
    CHECK(Swz::kLinePeriod == 8);
    for (int line = 0; line < 64; ++line) {
        std::set<int> seen;
        for (int e = 0; e < kPitch; ++e) {
            const int p = Swz::apply(line, e);
            CHECK(p >= 0 && p < kPitch);
            seen.insert(p);
            if (e % 16 == 0)
                for (int t = 1; t < 16; ++t) CHECK(Swz::apply(line, e + t) == p + t);
            CHECK(Swz::apply(line + 8, e) == p);
        }
        CHECK(int(seen.size()) == kPitch);
    }
    for (int line0 = 0; line0 < 64; line0 += 8) {
        for (int col0 = 0; col0 < kPitch; col0 += 16) {
            std::set<int> banks;
            for (int lane = 0; lane < 32; ++lane) {
                const int L = lane & 15, grp = lane >> 4;
                const int line = line0 + 4 * grp + (L >> 2), col = col0 + 4 * (L & 3);
                const int byte = (line * kPitch + Swz::apply(line, col)) * 2;
                for (int b = 0; b < 8; b += 4) banks.insert(((byte + b) / 4) % 64);
            }
            CHECK(int(banks.size()) == 64);
        }
    }
}

// The permutation for tiles whose lines are read 16 at a time in dealt order (lines 8 q + 4 h + r of a group of 32, h
// fixed per read): a bijection per line that keeps 16-byte units whole and repeats every 32 lines, and every pass of a
// 16-byte-per-lane read (16 lanes, one 16-byte unit column) touches 64 distinct banks.
static void test_swizzle_dealt() {
    constexpr int kPitch = 128;
    using Swz = tl::LdsSwizzleDealt<kPitch, 2>;
    CHECK(Swz::kLinePeriod == 32);
    for (int line = 0; line < 64; ++line) {
        std::set<int> seen;
        for (int e = 0; e < kPitch; ++e) {
            const int p = Swz::apply(line, e);
            CHECK(p >= 0 && p < kPitch);
            seen.insert(p);
            if (e % 8 == 0)
                for (int t = 1; t < 8; ++t) CHECK(Swz::apply(line, e + t) == p + t);
            CHECK(Swz::apply(line + 32, e) == p);
        }
        CHECK(int(seen.size()) == kPitch);
    }
    for (int pair = 0; pair < 2; ++pair)
        for (int h = 0; h < 2; ++h)
            for (int unit = 0; unit < 16; ++unit) {
                std::set<int> banks;
                for (int lane = 0; lane < 16; ++lane) {
                    const int line = 32 * pair + 8 * (lane / 4) + 4 * h + lane % 4;
                    const int byte = (line * kPitch + Swz::apply(line, unit * 8)) * 2;
                    for (int b = 0; b < 16; b += 4) banks.insert(((byte + b) / 4) % 64);
                }
                CHECK(int(banks.size()) == 64);
            }
}

// A ring whose stages are further apart than a tile (two rings interleaved in one allocation).
static void test_strided_ring() {
    using Shared = SharedTile<__half, tl::RowMajor<64, 128>, true>;
    using Packed = SharedRing<Shared, 5>;
    using Strided = SharedRing<Shared, 5, 2 * 64 * 128>;
    CHECK(Packed::kStageNumel == 64 * 128 && Packed::kBytes == 5 * 64 * 128 * 2);
    CHECK(Strided::kStageNumel == 2 * 64 * 128 && Strided::kStageBytes == 32768);
    CHECK(Strided::kBytes == (4 * 2 + 1) * 64 * 128 * 2);
    __half* base = nullptr;
    Strided ring(base);
    CHECK(ring.stage_data(3) == base + 3 * 2 * 64 * 128);
    CHECK(ring[2].data() == base + 2 * 2 * 64 * 128);
    CHECK(Strided::next(4) == 0 && Strided::next(1) == 2);
    // a tile with the transposing-read policy keeps it in the sub-tiles its iterator cuts
    using SharedV = SharedTile<__half, tl::RowMajor<64, 128>, true, tl::LdsSwizzleTr<128, 2>>;
    using Halves = STileIterator<SharedV, TileShape<32, 128>>;
    Halves halves(base);
    auto second = halves(1);
    CHECK(second.line0() == 32 && second.elem0() == 0);
    CHECK((std::is_same_v<typename decltype(second)::Swizzle, tl::LdsSwizzleTr<128, 2>>));
    CHECK(second.offset(1, 0) == 33 * 128 + tl::LdsSwizzleTr<128, 2>::apply(33, 0));
}

static void test_shared_tile_views() {
    using Shared = SharedTile<__half, tl::RowMajor<64, 128>, true>;
    using SIter = STileIterator<Shared, TileShape<64, 32>>;
    CHECK(SIter::sc0 == 1 && SIter::sc1 == 4);
    __half* base = nullptr;
    Shared whole(base);
    SIter it(base);
    // element (r, c) of chunk k is element (r, 32 k + c) of the parent, swizzle included
    for (int k = 0; k < 4; ++k) {
        auto sub = it(k);
        for (int r = 0; r < 64; r += 7)
            for (int c = 0; c < 32; ++c) CHECK(sub.offset(r, c) == whole.offset(r, 32 * k + c));
    }
    // offsets of a swizzled tile are a permutation of [0, numel)
    std::set<int> seen;
    for (int r = 0; r < 64; ++r)
        for (int c = 0; c < 128; ++c) seen.insert(whole.offset(r, c));
    CHECK(int(seen.size()) == 64 * 128 && *seen.rbegin() == 64 * 128 - 1);

    using SharedB = SharedTile<__half, tl::ColMajor<64, 32>, true>;
    using SIterB = STileIterator<SharedB, TileShape<16, 32>>;
    SharedB wb(base);
    SIterB itb(base);
    CHECK(SIterB::sc0 == 4 && SIterB::sc1 == 1);
    for (int k = 0; k < 4; ++k) {
        auto sub = itb(k);
        for (int r = 0; r < 16; ++r)
            for (int c = 0; c < 32; c += 5) CHECK(sub.offset(r, c) == wb.offset(16 * k + r, c));
    }
    // 2-D index and slices (left unimplemented by the reference)
    using SIter2 = STileIterator<Shared, TileShape<16, 32>>;
    SIter2 it2(base);
    CHECK(it2(2, 3).offset(1, 1) == whole.offset(33, 97));
    CHECK(it2(2, _)(3).offset(1, 1) == whole.offset(33, 97));
    CHECK(it2(_, 3)(2).offset(1, 1) == whole.offset(33, 97));
    // a plain tile is just pitched
    SharedTile<float, tl::RowMajor<16, 32>, false> plain((float*)nullptr);
    CHECK(plain.offset(3, 5) == 3 * 32 + 5);
}

static void test_pipelined_gemm_maps() {
    // LDS rows of 128 B, 16-byte chunk c of row r stored at chunk c ^ ((r / 2) % 8): any 16 consecutive
    // lanes of a 16x16x32 operand read (rows r0..r0+15, one k-chunk) must touch 16 distinct 16-byte bank slots
    for (int kk = 0; kk < 2; ++kk)
        for (int quad = 0; quad < 4; ++quad)
            for (int r0 = 0; r0 < 64; r0 += 16) {
                std::set<int> slots;
                for (int r = r0; r < r0 + 16; ++r) {
                    const int chunk = (4 * kk + quad) ^ ((r >> 1) & 7);
                    slots.insert(((r * 128 + chunk * 16) / 16) % 16);
                }
                CHECK(slots.size() == 16);
            }
    // workgroup -> tile map: a bijection; the 32 ids of one XCD (same id mod 8) cover a compact block
    for (int tiles : {16, 8, 12, 5}) {
        std::set<std::pair<int, int>> seen;
        for (int bid = 0; bid < tiles * tiles; ++bid) {
            int tm, tn;
            kernels::detail::xcd_tile_coords(bid, tiles, tiles, tm, tn);
            CHECK(tm >= 0 && tm < tiles && tn >= 0 && tn < tiles);
            seen.insert({tm, tn});
        }
        CHECK(int(seen.size()) == tiles * tiles);
    }
    // ... also for grids that are neither a multiple of 8 tiles nor of 4 rows: a bijection, and the ids of one XCD
    // stay inside a few row panels (a run of ceil(total / 8) positions spans at most that many / (4 tiles_n) + 2)
    for (int tiles_m = 1; tiles_m <= 33; ++tiles_m)
        for (int tiles_n : {1, 2, 3, 5, 9, 13, 16, 27, 32}) {
            std::set<std::pair<int, int>> seen;
            std::set<int> panels_of_xcd[8];
            for (int bid = 0; bid < tiles_m * tiles_n; ++bid) {
                int tm, tn;
                kernels::detail::xcd_tile_coords(bid, tiles_m, tiles_n, tm, tn);
                CHECK(tm >= 0 && tm < tiles_m && tn >= 0 && tn < tiles_n);
                seen.insert({tm, tn});
                panels_of_xcd[bid % 8].insert(tm / 4);
            }
            CHECK(int(seen.size()) == tiles_m * tiles_n);
            const int run = (tiles_m * tiles_n + 7) / 8;
            for (const auto& panels : panels_of_xcd) CHECK(int(panels.size()) <= run / (4 * tiles_n) + 2);
        }
    std::set<int> rows, cols;
    for (int bid = 3; bid < 256; bid += 8) {
        int tm, tn;
        kernels::detail::xcd_tile_coords(bid, 16, 16, tm, tn);
        rows.insert(tm);
        cols.insert(tn);
    }
    CHECK(rows.size() * cols.size() == 32);  // 32 tiles from a 4 x 8 block: 12 panels instead of 32
}

int main() {
    test_layout();
    test_gtile_iterator<true>();
    test_gtile_iterator<false>();
    test_tile_shape_and_regtile();
    test_swizzle<16, 2>(true);
    test_swizzle<32, 2>(true);
    test_swizzle<64, 2>(true);
    test_swizzle<128, 2>(true);
    test_swizzle<256, 2>(true);
    test_swizzle<48, 2>(false);
    test_swizzle<80, 2>(false);
    test_swizzle_tr<128>();
    test_swizzle_tr<64>();
    test_swizzle_tr8<128>();
    test_swizzle_tr8<64>();
    test_swizzle_dealt();
    test_strided_ring();
    test_swizzle<16, 4>(true);
    test_swizzle<32, 4>(true);
    test_swizzle<64, 4>(true);
    test_swizzle<256, 4>(true);
    test_swizzle<48, 4>(false);
    test_shared_tile_views();
    test_pipelined_gemm_maps();
    std::printf("%s (%d failed checks)\n", g_failed ? "FAILED" : "OK", g_failed);
    return g_failed ? 1 : 0;
}
