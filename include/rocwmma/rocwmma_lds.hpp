// gfx950 data paths between global memory, LDS and MFMA-ready fragments.
//
// Extension of the rocWMMA-style API (no counterpart in the reference, which moves macro
// tiles global -> VGPR -> (shuffle) -> LDS -> VGPR -> (shuffle), see reference
// samples/perf_hgemm.cpp:328-409).  On CDNA4 the same job is done with
//
//   * global_load_lds_dwordx4: each lane copies 16 bytes from global memory straight into
//     LDS (lane i of the issuing wave lands at ldsBase + 16*i) without touching VGPRs;
//   * LDS tiles whose 16-byte chunks are XOR-swizzled so that the ds_read_b128 of an MFMA
//     operand (16 or 32 consecutive rows, same K chunk) touches every bank once;
//   * ds_read_b64_tr_b16 for operands stored with the non-K dimension contiguous
//     (column-major A, row-major B): the transposing LDS read returns, to lane i of each
//     16-lane group, the i-th column of a 4 x 16 block whose rows the lanes addressed.
//
// Two LDS tile formats, both for a macro-tile operand of `Dim` rows/columns by 128 bytes of K
// (64 halves or 128 bytes) and both filled by whole-wave 1 KiB direct loads:
//
//   KMajorTile  -- one operand row per 128-byte LDS row (row-major A / col-major B).
//   DimMajorTile -- one K index per LDS row of Dim elements (col-major A / row-major B),
//                   16-bit elements only.
#ifndef ROCWMMA_LDS_HPP
#define ROCWMMA_LDS_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace lds
    {
        using LdsPtr    = __attribute__((address_space(3))) void*;
        using GlobalPtr = __attribute__((address_space(1))) const void*;

        // One wave copies 64 x 16 bytes: lane i fetches `src` (its own pointer) into
        // ldsBase + 16 * i.  ldsBase must be wave uniform.  Completion is tracked by vmcnt.
        ROCWMMA_DEVICE ROCWMMA_INLINE void asyncCopy16(void* ldsBase, const void* src)
        {
            __builtin_amdgcn_global_load_lds((GlobalPtr)src, (LdsPtr)ldsBase, 16, 0, 0);
        }

        // Waits until all of this wave's direct-to-LDS copies (and other vector memory loads)
        // have landed.  Follow with synchronize_workgroup() before other waves read the data.
        ROCWMMA_DEVICE ROCWMMA_INLINE void asyncCopyWait()
        {
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0), expcnt / lgkmcnt untouched
        }

        // ---------------------------------------------------------------------------------
        // K-major tile: Dim rows of 128 bytes; chunk c (16 bytes) of row r lives at chunk
        // position c ^ swz(r).  swz makes any 8 consecutive rows and any 16 consecutive rows
        // of one chunk column fall into distinct banks (32- and 64-bank views of the LDS).
        // ---------------------------------------------------------------------------------
        template <uint32_t Dim>
        struct KMajorTile
        {
            static constexpr uint32_t rowBytes  = 128u;
            static constexpr uint32_t chunks    = 8u;
            static constexpr uint32_t bytes     = Dim * rowBytes;
            static constexpr uint32_t waveLoads = bytes / 1024u; // whole-wave copies per tile

            ROCWMMA_HOST_DEVICE static constexpr uint32_t swz(uint32_t row)
            {
                return (row ^ (row >> 3)) & 7u;
            }
            ROCWMMA_HOST_DEVICE static constexpr uint32_t offset(uint32_t row, uint32_t chunk)
            {
                return row * rowBytes + ((chunk ^ swz(row)) << 4);
            }

            // Wave `waveIndex` of `WaveCount` issues its share of the copies of one tile.
            // `src` points at element (row 0, k 0) of the tile in global memory, rows
            // `ldBytes` apart, K contiguous.
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                asyncLoad(char* ldsTile, const char* src, uint32_t ldBytes, uint32_t waveIndex, uint32_t lane)
            {
                static_assert(waveLoads % WaveCount == 0u, "tile must split evenly over the waves");
                // a copy covers 8 rows; lane i owns LDS position (row i/8, chunk position i%8)
                const uint32_t rowInCopy = lane >> 3;
                const uint32_t pos       = lane & 7u;
#pragma unroll
                for(uint32_t i = 0; i < waveLoads / WaveCount; ++i)
                {
                    const uint32_t copy  = i * WaveCount + waveIndex;
                    const uint32_t row   = copy * 8u + rowInCopy;
                    const uint32_t chunk = pos ^ swz(row);
                    asyncCopy16(ldsTile + copy * 1024u, src + row * ldBytes + (chunk << 4));
                }
            }

            // Reads the operand of one 32-wide MFMA block: rows [row0, row0+32), K step `ks`.
            // KPackBytes = bytes of K each lane holds per MFMA (16, or 32 for wide fp8).
            template <uint32_t KPackBytes>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock32(void* regs, const char* ldsTile, uint32_t row0, uint32_t ks, uint32_t lane)
            {
                constexpr uint32_t perLane = KPackBytes / 16u;
                const uint32_t     row     = row0 + (lane & 31u);
                const uint32_t     first   = (ks * 2u + (lane >> 5)) * perLane;
#pragma unroll
                for(uint32_t j = 0; j < perLane; ++j)
                    reinterpret_cast<detail::u32x4*>(regs)[j]
                        = *reinterpret_cast<const detail::u32x4*>(ldsTile + offset(row, first + j));
            }
        };

        // ---------------------------------------------------------------------------------
        // Dim-major tile (16-bit elements): 64 LDS rows (one per K index) of Dim elements.
        // Rows are cut into 32-byte segments (16 elements); segment s of K row k lives at
        // segment position s ^ swz(k), which spreads the four K rows and two segments a
        // half-wave touches in one transposing read over all banks.
        // ---------------------------------------------------------------------------------
        template <uint32_t Dim>
        struct DimMajorTile
        {
            static_assert(Dim % 128u == 0u, "tile rows must hold at least eight 32-byte segments");
            static constexpr uint32_t kRows     = 64u;
            static constexpr uint32_t rowBytes  = Dim * 2u;
            static constexpr uint32_t bytes     = kRows * rowBytes;
            static constexpr uint32_t waveLoads = bytes / 1024u;
            static constexpr uint32_t slotsPerRow = rowBytes / 16u; // 16-byte copy slots per K row

            ROCWMMA_HOST_DEVICE static constexpr uint32_t swz(uint32_t k)
            {
                return (k & 3u) << 1;
            }
            ROCWMMA_HOST_DEVICE static constexpr uint32_t offset(uint32_t k, uint32_t seg)
            {
                return k * rowBytes + ((seg ^ swz(k)) << 5);
            }

            // `src` points at element (k 0, dim 0) of the tile, K rows `ldBytes` apart.
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                asyncLoad(char* ldsTile, const char* src, uint32_t ldBytes, uint32_t waveIndex, uint32_t lane)
            {
                static_assert(waveLoads % WaveCount == 0u, "tile must split evenly over the waves");
                static_assert(slotsPerRow >= 64u ? (slotsPerRow % 64u == 0u) : (64u % slotsPerRow == 0u),
                              "copy must cover whole or even parts of K rows");
#pragma unroll
                for(uint32_t i = 0; i < waveLoads / WaveCount; ++i)
                {
                    const uint32_t copy = i * WaveCount + waveIndex;
                    const uint32_t slot = copy * 64u + lane; // global 16-byte slot index in the tile
                    const uint32_t k    = slot / slotsPerRow;
                    const uint32_t pos  = slot % slotsPerRow; // physical slot within the row
                    const uint32_t seg  = (pos >> 1) ^ swz(k); // logical 32-byte segment
                    asyncCopy16(ldsTile + copy * 1024u, src + k * ldBytes + (seg << 5) + ((pos & 1u) << 4));
                }
            }

            // Operand of one 32-wide MFMA block with 8 K values per lane (v_mfma_*_32x32x16):
            // lane l ends up with dim = dim0 + l % 32 and k = ks*16 + (l/32)*8 + 0..7.
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock32(void* regs, const char* ldsTile, uint32_t dim0, uint32_t ks, uint32_t lane)
            {
                typedef short s16x4 __attribute__((ext_vector_type(4)));
                using LdsVec = __attribute__((address_space(3))) s16x4*;
                const uint32_t group  = lane >> 4; // 16-lane group
                const uint32_t s      = lane & 15u; // source index inside the group
                const uint32_t seg    = (dim0 >> 4) + (group & 1u);
                const uint32_t kBase  = ks * 16u + (group >> 1) * 8u + (s >> 2);
                const uint32_t inSeg  = (s & 3u) << 3; // 4 elements = 8 bytes per source lane
#pragma unroll
                for(uint32_t kk = 0; kk < 2u; ++kk)
                {
                    const uint32_t k = kBase + kk * 4u;
                    reinterpret_cast<s16x4*>(regs)[kk]
                        = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsVec)(ldsTile + offset(k, seg) + inSeg));
                }
            }
        };

    } // namespace lds
} // namespace rocwmma

#endif // ROCWMMA_LDS_HPP
