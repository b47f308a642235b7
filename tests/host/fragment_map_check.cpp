// Host enumeration of the fragment-to-register maps (include/rocwmma/internal/fragment_map.hpp).
// For each map: every (lane, element) pair must name a distinct matrix element, together they
// must cover the block exactly, K runs must be contiguous, and the map must agree with the
// operand layout of the gfx950 MFMA instruction it feeds (one lane = one row, runs of K;
// accumulators = 4-column runs of one row).  Exit code 0 = all checks passed.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/rocwmma/internal/fragment_map.hpp"

using namespace rocwmma::detail;

static int failures = 0;
#define CHECK(cond, ...)                    \
    do                                      \
    {                                       \
        if(!(cond))                         \
        {                                   \
            std::printf("FAIL: " __VA_ARGS__); \
            std::printf("\n");              \
            ++failures;                     \
        }                                   \
    } while(0)

template <uint32_t Dim, uint32_t K, uint32_t Tile, PackClass C>
void checkInput(const char* name, uint32_t expectKPack)
{
    using M = InputMap<Dim, K, Tile, C>;
    CHECK(M::kpack == expectKPack, "%s: kpack %u != %u", name, M::kpack, expectKPack);
    std::vector<int> seen(Dim * K, 0);
    for(uint32_t lane = 0; lane < 64; ++lane)
        for(uint32_t e = 0; e < M::size; ++e)
        {
            uint32_t d = M::dimOf(e, lane), k = M::kOf(e, lane);
            CHECK(d < Dim && k < K, "%s: out of range lane %u e %u -> (%u,%u)", name, lane, e, d, k);
            if(d < Dim && k < K)
                seen[d * K + k]++;
            // runs of kpack elements are contiguous in K and stay on one row
            if(e % M::kpack)
                CHECK(M::dimOf(e - 1, lane) == d && M::kOf(e - 1, lane) + 1 == k, "%s: run broken", name);
            // MFMA operand rule: lane % tile selects the row inside the block, lane / tile the K group
            CHECK(d % Tile == lane % Tile, "%s: row rule", name);
            CHECK((k % M::kstep) / M::kpack == lane / Tile, "%s: k-group rule", name);
        }
    for(uint32_t i = 0; i < Dim * K; ++i)
        CHECK(seen[i] == 1, "%s: element %u covered %d times", name, i, seen[i]);
}

template <uint32_t BM, uint32_t BN, uint32_t Tile>
void checkAcc(const char* name)
{
    using M = AccMap<BM, BN, Tile>;
    std::vector<int> seen(BM * BN, 0);
    for(uint32_t lane = 0; lane < 64; ++lane)
        for(uint32_t e = 0; e < M::size; ++e)
        {
            uint32_t r = M::rowOf(e, lane), c = M::colOf(e, lane);
            CHECK(r < BM && c < BN, "%s: out of range", name);
            if(r < BM && c < BN)
                seen[r * BN + c]++;
            if(e % 4)
                CHECK(M::rowOf(e - 1, lane) == r && M::colOf(e - 1, lane) + 1 == c, "%s: 4-run broken", name);
            CHECK(c % 4 == e % 4, "%s: runs must start on 4-column boundaries", name);
            // transposed MFMA result: lane % tile is the row inside the block
            CHECK(r % Tile == lane % Tile, "%s: row rule", name);
            // inside a block, the instruction's register index i maps to 8*(i/4) + 4*(lane/tile) + i%4
            uint32_t i  = e % M::perBlock;
            uint32_t cc = (Tile == 16 ? 0 : 8 * (i / 4)) + 4 * (lane / Tile) + i % 4;
            CHECK(c % Tile == cc, "%s: column rule", name);
        }
    for(uint32_t i = 0; i < BM * BN; ++i)
        CHECK(seen[i] == 1, "%s: element %u covered %d times", name, i, seen[i]);
}

// 64-bit accumulators: v_mfma_f64_16x16x4_f64 puts register i of lane l on row (l / 16) + 4 i and column
// l % 16 of its result; with the multiplicands swapped that is row l % 16, column (l / 16) + 4 i of D.
template <uint32_t BM, uint32_t BN>
void checkAccStrided(const char* name)
{
    using M = AccMapStrided<BM, BN>;
    std::vector<int> seen(BM * BN, 0);
    CHECK(M::size * 64 == BM * BN && M::nruns == M::size && M::runLen == 1, "%s: sizes", name);
    for(uint32_t lane = 0; lane < 64; ++lane)
        for(uint32_t e = 0; e < M::size; ++e)
        {
            uint32_t r = M::rowOf(e, lane), c = M::colOf(e, lane);
            CHECK(r < BM && c < BN, "%s: out of range", name);
            if(r < BM && c < BN)
                seen[r * BN + c]++;
            CHECK(r % 16 == lane % 16, "%s: row rule", name);
            CHECK(c % 16 == lane / 16 + 4 * (e % 4), "%s: column rule", name);
            CHECK(r / 16 == (e / 4) / M::nbj && c / 16 == (e / 4) % M::nbj, "%s: tile order", name);
        }
    for(uint32_t i = 0; i < BM * BN; ++i)
        CHECK(seen[i] == 1, "%s: element %u covered %d times", name, i, seen[i]);
}

int main()
{
    // K packing picks the widest gfx950 instruction that divides BlockK
    checkInput<16, 32, 16, PackClass::Bits16>("f16 16x32 t16", 8); // 16x16x32
    checkInput<16, 16, 16, PackClass::Bits16>("f16 16x16 t16", 4); // 16x16x16
    checkInput<16, 64, 16, PackClass::Bits16>("f16 16x64 t16", 8);
    checkInput<32, 16, 32, PackClass::Bits16>("f16 32x16 t32", 8); // 32x32x16
    checkInput<32, 8, 32, PackClass::Bits16>("f16 32x8 t32", 4); // 32x32x8
    checkInput<128, 16, 32, PackClass::Bits16>("f16 128x16 t32", 8);
    checkInput<256, 64, 32, PackClass::Bits16>("f16 256x64 t32", 8);
    checkInput<64, 16, 16, PackClass::Bits16>("f16 64x16 t16", 4);
    checkInput<16, 64, 16, PackClass::Int8>("i8 16x64 t16", 16); // 16x16x64
    checkInput<16, 32, 16, PackClass::Int8>("i8 16x32 t16", 8); // 16x16x32
    checkInput<32, 32, 32, PackClass::Int8>("i8 32x32 t32", 16); // 32x32x32
    checkInput<32, 16, 32, PackClass::Int8>("i8 32x16 t32", 8);
    checkInput<16, 128, 16, PackClass::Fp8>("f8 16x128 t16", 16); // 16x16x128: two 16-byte runs per lane
    checkInput<16, 64, 16, PackClass::Fp8>("f8 16x64 t16", 8); // 2 x 16x16x32 (no 16-byte fp8 operand)
    checkInput<16, 32, 16, PackClass::Fp8>("f8 16x32 t16", 8);
    checkInput<32, 64, 32, PackClass::Fp8>("f8 32x64 t32", 16); // 32x32x64: two 16-byte runs per lane
    checkInput<32, 32, 32, PackClass::Fp8>("f8 32x32 t32", 8);
    checkInput<32, 16, 32, PackClass::Fp8>("f8 32x16 t32", 8);
    checkInput<16, 16, 16, PackClass::Bits32>("f32 16x16 t16", 1); // 16x16x4
    checkInput<32, 16, 32, PackClass::Bits32>("f32 32x16 t32", 1); // 32x32x2
    checkInput<16, 4, 16, PackClass::Bits16>("f16 16x4 t16", 1);

    checkAcc<16, 16, 16>("acc 16x16");
    checkAcc<32, 32, 32>("acc 32x32");
    checkAcc<64, 64, 32>("acc 64x64");
    checkAcc<48, 16, 16>("acc 48x16");
    checkAcc<32, 64, 32>("acc 32x64");
    checkAcc<128, 128, 32>("acc 128x128");
    checkAccStrided<16, 16>("f64 acc 16x16");
    checkAccStrided<32, 32>("f64 acc 32x32");
    checkAccStrided<64, 16>("f64 acc 64x16");
    checkInput<16, 4, 16, PackClass::Other>("f64 16x4 t16", 1); // 16x16x4
    checkInput<32, 16, 16, PackClass::Other>("f64 32x16 t16", 1);
    // blocks with an edge of 8: load / store only
    checkInput<8, 32, 8, PackClass::Bits16>("f16 8x32 t8", 4);
    checkInput<8, 256, 8, PackClass::Bits16>("f16 8x256 t8", 8);
    checkInput<8, 64, 8, PackClass::Int8>("i8 8x64 t8", 8);
    checkInput<8, 32, 8, PackClass::Fp8>("f8 8x32 t8", 4);
    checkInput<8, 128, 8, PackClass::Other>("f64 8x128 t8", 1);
    checkAcc<32, 8, 32>("acc 32x8");
    checkAcc<256, 8, 32>("acc 256x8");

    CHECK(mmaTileDim(32, 32) == 32 && mmaTileDim(64, 32) == 32 && mmaTileDim(32, 16) == 16 && mmaTileDim(16, 16) == 16
              && mmaTileDim(128, 1) == 16 && inputTileDim(1, 8, 8) == 8 && inputTileDim(32, 32, 32) == 32
              && inputTileDim(64, 1, 64) == 16 && accTileRows(64, 8) == 32 && accTileRows(64, 32) == 32
              && accTileRows(16, 32) == 16,
          "tile choice");
    if(failures)
    {
        std::printf("%d failures\n", failures);
        return 1;
    }
    std::printf("fragment maps OK\n");
    return 0;
}
