// Register <-> memory movers for fragments (global memory or LDS, through generic pointers).
//
// A fragment is a sequence of "items": for input fragments an item is one MFMA operand
// (kpack elements contiguous in K, see fragment_map.hpp); for accumulators an item is a run
// of four consecutive columns of one row (a single element for 64-bit accumulators).  Items whose elements are contiguous in memory
// (K-contiguous operands; row-major accumulators) move as one 2..32-byte vector access.
// Input items of 16 bytes per lane whose K index is NOT the contiguous one (col-major matrix_a,
// row-major matrix_b) also move as 16-byte vectors: every lane accesses one memory row (16 bytes along
// the contiguous dimension, one K index) and a transpose inside groups of 8 lanes (16-bit elements) or
// 16 lanes (8-bit elements) converts between that and the register order (see LaneTranspose).
// Column-major accumulator runs move as one vector after a 4 x 4 transpose inside quads of lanes.
// Everything else moves element by element.
//
// The same walk serves the cooperative API.  Wave w of a pool of W waves owns the fragment's
// elements [w * size / W, (w + 1) * size / W) (a blocked, not a strided, assignment) and keeps them in
// its FIRST size / W register elements; the rest of its fragment is untouched.  With Items % W == 0 that
// is a run of whole items; with more waves than items (W % Items == 0) an item is cut into W / Items
// equal pieces.  Because a share is "the first size / W register elements <-> the w-th size / W-th of the
// fragment", a cooperative fragment may be reinterpreted as another fragment type with the same element
// count (an LDS "register file" view, say) and stored cooperatively with the same (w, W): every wave then
// writes what it read, whatever the item sizes of the two types.  Other wave counts (3 waves, 4 items)
// fall back to ceil(Items / W) whole items per wave, which agrees only between types with equal item
// sizes.  Keeping a share at the front of the registers keeps every register index a compile-time
// constant without any branch on the wave index (with shares at their ordinary positions, behind
// "if (w == i)" branches, the reference's perf_hgemm sample ran three times slower: the compiler merged
// the branches into one body with a computed register index and the fragments went to scratch memory).
// (rocWMMA's engines for the same job: reference library/include/rocwmma/internal/
// opaque_load.hpp:65-159, opaque_store.hpp:56-135, coop_load.hpp:43-218, coop_store.hpp:43-217.)
//
// Alignment contract: a vector access of B bytes needs its address aligned to min(B, 16).
// That holds when the tile origin and the leading dimension are multiples of 16 bytes (in either
// orientation: the dim-major vector path reads 16 bytes along the contiguous dimension).
#ifndef ROCWMMA_FRAGMENT_IO_HPP
#define ROCWMMA_FRAGMENT_IO_HPP

#include "fragment_map.hpp"
#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <uint32_t Bytes>
        ROCWMMA_DEVICE ROCWMMA_INLINE void copyBytes(void* dst, const void* src)
        {
            if constexpr(Bytes % 16u == 0u)
            {
#pragma unroll
                for(uint32_t i = 0; i < Bytes / 16u; ++i)
                    reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
            }
            else if constexpr(Bytes == 8u)
                *reinterpret_cast<u32x2*>(dst) = *reinterpret_cast<const u32x2*>(src);
            else if constexpr(Bytes == 4u)
                *reinterpret_cast<u32x1*>(dst) = *reinterpret_cast<const u32x1*>(src);
            else if constexpr(Bytes == 2u)
                *reinterpret_cast<u16x1*>(dst) = *reinterpret_cast<const u16x1*>(src);
            else
            {
                static_assert(Bytes == 1u, "unsupported vector width");
                *reinterpret_cast<u8x1*>(dst) = *reinterpret_cast<const u8x1*>(src);
            }
        }


        // ---- transposes across lanes -----------------------------------------------------
        // Four registers (16 bytes) per lane.  transpose8x8Halves: inside every group of 8 consecutive
        // lanes, lane r holds row r of an 8 x 8 matrix of 16-bit elements; afterwards lane c holds column c.
        // transpose16x16Bytes: the same for 16 x 16 bytes in groups of 16 lanes.  Both are their own
        // inverse.  Each is a butterfly: stage b swaps bit b of the lane index with bit b of the element
        // index, i.e. a lane keeps the elements whose bit b equals its own and trades the others with lane
        // ^ (1 << b).  Whole registers are traded with DPP row shifts whose bank mask picks the receiving
        // half of the lanes (distances 4 and 8), or with a quad permute and selects (distance 2 inside a
        // quad); halves and bytes of registers with a quad permute followed by v_perm_b32.
        // (rocWMMA reaches the same end with its AOS <-> SOA register transforms, reference
        // library/include/rocwmma/internal/transforms.hpp and io_layout.hpp:160-226.)
        struct LaneTranspose
        {
            static constexpr int QuadXor1 = 0xB1; // quad_perm:[1,0,3,2]
            static constexpr int QuadXor2 = 0x4E; // quad_perm:[2,3,0,1]
            static constexpr int RowShl4 = 0x104, RowShr4 = 0x114, RowShl8 = 0x108, RowShr8 = 0x118;

            template <int Ctrl, int BankMask>
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t dpp(uint32_t keep, uint32_t src)
            {
                return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
                    static_cast<int>(keep), static_cast<int>(src), Ctrl, 0xF, BankMask, false));
            }

            // registers (a, b) <-> (c, d) between lanes `Shift` apart: the lower lane of a pair ends up
            // with the upper lane's (a, b) in its (c, d); the upper lane with the lower lane's (c, d) in
            // its (a, b).  LowerBanks: the banks (groups of 4 lanes of a row of 16) of the lower lanes.
            template <int Shl, int Shr, int LowerBanks>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                tradeRegisters(uint32_t& a, uint32_t& b, uint32_t& c, uint32_t& d)
            {
                const uint32_t nc = dpp<Shl, LowerBanks>(c, a);
                const uint32_t nd = dpp<Shl, LowerBanks>(d, b);
                const uint32_t na = dpp<Shr, 0xF & ~LowerBanks>(a, c);
                const uint32_t nb = dpp<Shr, 0xF & ~LowerBanks>(b, d);
                a = na, b = nb, c = nc, d = nd;
            }

            // value of lane `QuadPerm(lane)` for every lane (nothing kept: no tie to an old register)
            template <int QuadPerm>
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t quad(uint32_t src)
            {
                return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(src), QuadPerm, 0xF, 0xF, true));
            }

            // halves or bytes of every register (which ones: the v_perm_b32 selectors of the lower and the
            // upper lane) between the lanes of a quad that differ in `LaneBit`
            template <int QuadPerm, uint32_t LaneBit, uint32_t LowerSel, uint32_t UpperSel>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void tradeWithinRegisters(uint32_t (&x)[4], uint32_t lane)
            {
                const uint32_t sel = (lane & LaneBit) ? UpperSel : LowerSel;
#pragma unroll
                for(uint32_t d = 0; d < 4u; ++d)
                {
                    x[d] = __builtin_amdgcn_perm(quad<QuadPerm>(x[d]), x[d], sel);
                }
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void transpose8x8Halves(uint32_t (&x)[4], uint32_t lane)
            {
                // element bit 2 = register bit 1, lane bit 2: lanes 0-3 and 8-11 of a row are the lower ones
                tradeRegisters<RowShl4, RowShr4, 0x5>(x[0], x[1], x[2], x[3]);
                // element bit 1 = register bit 0, lane bit 1 (inside a quad)
                // (written so that each select can take its permuted operand as a DPP source)
                const bool     upper = (lane & 2u) != 0u;
                const uint32_t p0 = quad<QuadXor2>(x[0]), p1 = quad<QuadXor2>(x[1]);
                const uint32_t p2 = quad<QuadXor2>(x[2]), p3 = quad<QuadXor2>(x[3]);
                x[0] = upper ? p1 : x[0];
                x[1] = upper ? x[1] : p0;
                x[2] = upper ? p3 : x[2];
                x[3] = upper ? x[3] : p2;
                // element bit 0 = half of a register, lane bit 0
                tradeWithinRegisters<QuadXor1, 1u, 0x05040100u, 0x03020706u>(x, lane);
            }

            // 4 x 4 transposes inside quads of lanes (lane q holds row q; afterwards column q), for elements
            // of 4, 2 and 1 bytes: 4, 2 and 1 registers per lane.
            ROCWMMA_DEVICE static ROCWMMA_INLINE void transpose4x4(uint32_t (&x)[4], uint32_t lane)
            {
                bool           upper = (lane & 2u) != 0u;
                const uint32_t p0 = quad<QuadXor2>(x[0]), p1 = quad<QuadXor2>(x[1]);
                const uint32_t p2 = quad<QuadXor2>(x[2]), p3 = quad<QuadXor2>(x[3]);
                x[0] = upper ? p2 : x[0];
                x[1] = upper ? p3 : x[1];
                x[2] = upper ? x[2] : p0;
                x[3] = upper ? x[3] : p1;
                upper = (lane & 1u) != 0u;
                const uint32_t q0 = quad<QuadXor1>(x[0]), q1 = quad<QuadXor1>(x[1]);
                const uint32_t q2 = quad<QuadXor1>(x[2]), q3 = quad<QuadXor1>(x[3]);
                x[0] = upper ? q1 : x[0];
                x[1] = upper ? x[1] : q0;
                x[2] = upper ? q3 : x[2];
                x[3] = upper ? x[3] : q2;
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void transpose4x4(uint32_t (&x)[2], uint32_t lane)
            {
                const bool     upper = (lane & 2u) != 0u;
                const uint32_t p0 = quad<QuadXor2>(x[0]), p1 = quad<QuadXor2>(x[1]);
                x[0] = upper ? p1 : x[0];
                x[1] = upper ? x[1] : p0;
                const uint32_t sel = (lane & 1u) ? 0x03020706u : 0x05040100u;
                x[0] = __builtin_amdgcn_perm(quad<QuadXor1>(x[0]), x[0], sel);
                x[1] = __builtin_amdgcn_perm(quad<QuadXor1>(x[1]), x[1], sel);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void transpose4x4(uint32_t (&x)[1], uint32_t lane)
            {
                x[0] = __builtin_amdgcn_perm(quad<QuadXor2>(x[0]), x[0], (lane & 2u) ? 0x03020706u : 0x05040100u);
                x[0] = __builtin_amdgcn_perm(quad<QuadXor1>(x[0]), x[0], (lane & 1u) ? 0x03070105u : 0x06020400u);
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void transpose16x16Bytes(uint32_t (&x)[4], uint32_t lane)
            {
                tradeRegisters<RowShl8, RowShr8, 0x3>(x[0], x[1], x[2], x[3]); // byte bit 3, lane bit 3
                tradeRegisters<RowShl4, RowShr4, 0x5>(x[0], x[2], x[1], x[3]); // byte bit 2, lane bit 2
                tradeWithinRegisters<QuadXor2, 2u, 0x05040100u, 0x03020706u>(x, lane); // byte bit 1, lane bit 1
                tradeWithinRegisters<QuadXor1, 1u, 0x06020400u, 0x03070105u>(x, lane); // byte bit 0, lane bit 0
            }
        };

        // ---- LDS reads that transpose ------------------------------------------------------
        // True when the generic pointer points into LDS (folds to a constant wherever the compiler has
        // inferred the address space, which is the usual case after inlining).  The answer is taken from
        // the first active lane, so a branch on it is a scalar branch: every lane of a wave passes the same
        // tile pointer, but the compiler cannot always see that, and the transposing LDS reads must not be
        // reached under a lane mask (they execute whatever the mask says and would overwrite the
        // destination registers of the other branch).
        ROCWMMA_DEVICE ROCWMMA_INLINE bool isLdsPointer(const void* p)
        {
#if defined(__HIP_DEVICE_COMPILE__)
            return __builtin_amdgcn_readfirstlane(
                       static_cast<int>(__builtin_amdgcn_is_shared((const __attribute__((address_space(0))) void*)p)))
                   != 0;
#else
            (void)p;
            return false;
#endif
        }

        // ds_read_b64_tr_b16: inside a group of 16 lanes, lane s addresses 8 bytes (4 consecutive dims
        // (s % 4) * 4 .. + 3 of memory row s / 4); lane t receives dim t of the 4 rows.
        // ds_read_b64_tr_b8: lane s addresses 8 bytes (dims (s % 2) * 8 .. + 7 of memory row s / 2); lane t
        // receives dim t of the 8 rows.  Either way one read yields 8 bytes of consecutive K for one dim
        // out of a block of 16 consecutive dims, which is the register order of input fragments.
        template <typename DataT>
        struct LdsTransposedRead
        {
            static constexpr uint32_t RowsPerRead = 8u / sizeof(DataT); // K indices per read: 4 or 8
            static constexpr uint32_t LanesPerRow = 16u / RowsPerRead; // 4 or 2

            // `block`: first of the 16 dims at the first K index; the lane receives dim lane % 16,
            // Reads * RowsPerRead consecutive K indices.
            template <uint32_t Reads>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void read(DataT* reg, const DataT* block, uint32_t ld, uint32_t lane)
            {
#if defined(__HIP_DEVICE_COMPILE__)
                const uint32_t s = lane & 15u;
                const DataT*   p = block + (s / LanesPerRow) * ld + (s % LanesPerRow) * (16u / LanesPerRow);
#pragma unroll
                for(uint32_t r = 0; r < Reads; ++r)
                {
                    const DataT* q = p + r * RowsPerRead * ld;
                    if constexpr(sizeof(DataT) == 2u)
                    {
                        typedef short s16x4 __attribute__((ext_vector_type(4)));
                        const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)q);
                        copyBytes<8u>(reg + r * RowsPerRead, &v);
                    }
                    else
                    {
                        typedef int i32x2 __attribute__((ext_vector_type(2)));
                        const i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)q);
                        copyBytes<8u>(reg + r * RowsPerRead, &v);
                    }
                }
#else
                (void)reg, (void)block, (void)ld, (void)lane;
#endif
            }
        };

        // ---- input fragments -------------------------------------------------------------
        // KContiguous: memory offset of (dim, k) is dim * ld + k  (matrix_a row_major,
        // matrix_b col_major); otherwise k * ld + dim.
        template <typename Map, typename DataT, bool KContiguous>
        struct InputIO
        {
            static constexpr uint32_t Items     = Map::nchunks;
            static constexpr uint32_t ItemElems = Map::kpack;

            // Dim-major memory, whole items of 16-byte multiples per lane on 16- or 32-wide tiles: a group
            // of GroupLanes lanes (one K run each, consecutive dims) covers GroupLanes K indices x 16 bytes
            // of consecutive dims, which the lanes access as one memory row each.
            static constexpr uint32_t GroupLanes = 16u / sizeof(DataT); // 8 (16-bit), 16 (8-bit)
#ifndef ROCWMMA_AMD_DIM_MAJOR_VECTORS
#define ROCWMMA_AMD_DIM_MAJOR_VECTORS 1
#endif
#ifndef ROCWMMA_AMD_DIM_MAJOR_LDS_TR
#define ROCWMMA_AMD_DIM_MAJOR_LDS_TR 1
#endif
            static constexpr uint32_t Vectors
                = (ROCWMMA_AMD_DIM_MAJOR_VECTORS && !KContiguous && (sizeof(DataT) == 2u || sizeof(DataT) == 1u) && Map::tile >= 16u
                   && (Map::kpack * sizeof(DataT)) % 16u == 0u && Map::kpack % GroupLanes == 0u)
                      ? Map::kpack / GroupLanes
                      : 0u;

            // Loads from LDS: transposing reads of 8 bytes (items of at least 8 bytes per lane).
            static constexpr uint32_t LdsReads
                = (ROCWMMA_AMD_DIM_MAJOR_LDS_TR && !KContiguous && (sizeof(DataT) == 2u || sizeof(DataT) == 1u) && Map::tile >= 16u
                   && (Map::kpack * sizeof(DataT)) % 8u == 0u)
                      ? Map::kpack * sizeof(DataT) / 8u
                      : 0u;

            ROCWMMA_DEVICE static ROCWMMA_INLINE void transposeGroup(uint32_t (&w)[4], uint32_t lane)
            {
                if constexpr(sizeof(DataT) == 2u)
                    LaneTranspose::transpose8x8Halves(w, lane);
                else
                    LaneTranspose::transpose16x16Bytes(w, lane);
            }

            // Elements [first, first + Count) of item `item`; the whole item is <ItemElems>(.., 0u, ..).
            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadPart(DataT* reg, uint32_t item, uint32_t first, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane) + first;
                if constexpr(KContiguous)
                    copyBytes<Count * sizeof(DataT)>(reg, data + dim * ld + k);
                else
                {
                    if constexpr(Count == ItemElems && LdsReads > 0u)
                    {
                        if(isLdsPointer(data))
                        {
                            LdsTransposedRead<DataT>::template read<LdsReads>(reg, data + k * ld + (dim - (lane & 15u)), ld, lane);
                            return;
                        }
                    }
                    if constexpr(Count == ItemElems && Vectors > 0u)
                    {
#pragma unroll
                        for(uint32_t v = 0; v < Vectors; ++v)
                        {
                            uint32_t w[4];
                            copyBytes<16u>(w, data + (k + v * GroupLanes + (lane % GroupLanes)) * ld + (dim - lane % GroupLanes));
                            transposeGroup(w, lane);
                            copyBytes<16u>(reg + v * GroupLanes, w);
                        }
                    }
                    else
                    {
#pragma unroll
                        for(uint32_t j = 0; j < Count; ++j)
                            copyBytes<sizeof(DataT)>(reg + j, data + (k + j) * ld + dim);
                    }
                }
            }

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storePart(const DataT* reg, uint32_t item, uint32_t first, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t dim = Map::chunkDim(item, lane);
                const uint32_t k   = Map::chunkK(item, lane) + first;
                if constexpr(KContiguous)
                    copyBytes<Count * sizeof(DataT)>(data + dim * ld + k, reg);
                else
                {
                    // (stores to LDS stay element-wise: 2-byte LDS writes cost less than the transpose)
                    if constexpr(Count == ItemElems && Vectors > 0u)
                    {
#ifndef ROCWMMA_AMD_DIM_MAJOR_LDS_VECTOR_STORES
#define ROCWMMA_AMD_DIM_MAJOR_LDS_VECTOR_STORES 0
#endif
                        if(ROCWMMA_AMD_DIM_MAJOR_LDS_VECTOR_STORES || !isLdsPointer(data))
                        {
#pragma unroll
                            for(uint32_t v = 0; v < Vectors; ++v)
                            {
                                uint32_t w[4];
                                copyBytes<16u>(w, reg + v * GroupLanes);
                                transposeGroup(w, lane);
                                copyBytes<16u>(data + (k + v * GroupLanes + (lane % GroupLanes)) * ld + (dim - lane % GroupLanes), w);
                            }
                            return;
                        }
                    }
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(data + (k + j) * ld + dim, reg + j);
                }
            }
        };

        // ---- accumulator fragments -------------------------------------------------------
        template <typename Map, typename DataT, bool RowMajor>
        struct AccIO
        {
            static constexpr uint32_t Items     = Map::nruns;
            static constexpr uint32_t ItemElems = Map::runLen; // 4 (1 for 64-bit accumulators)

            // Column-major memory: the four lanes of a quad own the same four columns of four consecutive
            // rows, so a 4 x 4 transpose inside the quad turns "four columns of my row" into "four rows of one
            // column", which is contiguous: one 16 / 8 / 4-byte access instead of four element accesses.
#ifndef ROCWMMA_AMD_COL_MAJOR_ACC_VECTORS
#define ROCWMMA_AMD_COL_MAJOR_ACC_VECTORS 1
#endif
            static constexpr bool     QuadVectors = ROCWMMA_AMD_COL_MAJOR_ACC_VECTORS && !RowMajor && ItemElems == 4u
                                                && (sizeof(DataT) == 4u || sizeof(DataT) == 2u || sizeof(DataT) == 1u);
            static constexpr uint32_t QuadWords = QuadVectors ? sizeof(DataT) : 1u; // registers per run

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadPart(DataT* reg, uint32_t item, uint32_t first, const DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane) + first;
                if constexpr(RowMajor)
                    copyBytes<Count * sizeof(DataT)>(reg, data + row * ld + col);
                else if constexpr(QuadVectors && Count == ItemElems)
                {
                    uint32_t w[QuadWords];
                    copyBytes<4u * sizeof(DataT)>(w, data + (col + (lane & 3u)) * ld + (row - (lane & 3u)));
                    LaneTranspose::transpose4x4(w, lane);
                    copyBytes<4u * sizeof(DataT)>(reg, w);
                }
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(reg + j, data + (col + j) * ld + row);
                }
            }

            template <uint32_t Count>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storePart(const DataT* reg, uint32_t item, uint32_t first, DataT* data, uint32_t ld, uint32_t lane)
            {
                const uint32_t row = Map::runRow(item, lane);
                const uint32_t col = Map::runCol(item, lane) + first;
                if constexpr(RowMajor)
                    copyBytes<Count * sizeof(DataT)>(data + row * ld + col, reg);
                else if constexpr(QuadVectors && Count == ItemElems)
                {
                    uint32_t w[QuadWords];
                    copyBytes<4u * sizeof(DataT)>(w, reg);
                    LaneTranspose::transpose4x4(w, lane);
                    copyBytes<4u * sizeof(DataT)>(data + (col + (lane & 3u)) * ld + (row - (lane & 3u)), w);
                }
                else
                {
#pragma unroll
                    for(uint32_t j = 0; j < Count; ++j)
                        copyBytes<sizeof(DataT)>(data + (col + j) * ld + row, reg + j);
                }
            }
        };

        // ---- whole-fragment and cooperative drivers --------------------------------------
        // Register positions are compile-time constants everywhere; a wave's index only enters address
        // arithmetic (which item, which piece), never a register index and never a branch around code that
        // differs in nothing but its registers (the compiler merges such branches into one body with a
        // computed register index, and the fragment then lives in scratch memory).
        template <typename IO, typename DataT>
        struct FragmentMover
        {
            static constexpr uint32_t Items     = IO::Items; // work items of the whole fragment
            static constexpr uint32_t ItemElems = IO::ItemElems;
            static constexpr uint32_t MaxWaves  = 16u; // 1024 threads per workgroup

            // `reg`: where the part's first element lives in registers
            template <bool Load, uint32_t Count, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                part(Reg* reg, uint32_t item, uint32_t first, Ptr* data, uint32_t ld, uint32_t lane)
            {
                if constexpr(Load)
                    IO::template loadPart<Count>(reg, item, first, data, ld, lane);
                else
                    IO::template storePart<Count>(reg, item, first, data, ld, lane);
            }

            template <bool Load, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void whole(Reg* x, Ptr* data, uint32_t ld)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
#pragma unroll
                for(uint32_t item = 0; item < Items; ++item)
                    part<Load, ItemElems>(x + item * ItemElems, item, 0u, data, ld, lane);
            }

            // Wave count known at compile time.
            template <bool Load, uint32_t WaveCount, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void shared(Reg* x, Ptr* data, uint32_t ld, uint32_t waveIndex)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                if constexpr(WaveCount > Items && WaveCount % Items == 0u && ItemElems % (WaveCount / Items) == 0u)
                {
                    // one piece of one item per wave, in its first registers
                    constexpr uint32_t pieces = WaveCount / Items, count = ItemElems / pieces;
                    if(waveIndex < WaveCount)
                        part<Load, count>(x, waveIndex / pieces, (waveIndex % pieces) * count, data, ld, lane);
                }
                else
                {
                    // items [w * per, (w + 1) * per) in register slots 0 .. per - 1
                    constexpr uint32_t per = (Items + WaveCount - 1u) / WaveCount;
#pragma unroll
                    for(uint32_t s = 0; s < per; ++s)
                    {
                        const uint32_t item = waveIndex * per + s;
                        if(Items % WaveCount == 0u ? waveIndex < WaveCount : item < Items)
                            part<Load, ItemElems>(x + s * ItemElems, item, 0u, data, ld, lane);
                    }
                }
            }

            // One piece of `Count` elements per wave, for a wave count only known at run time: tried for
            // every piece size an item can be cut into with at most MaxWaves waves.
            template <bool Load, uint32_t Count, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                pieces(Reg* x, Ptr* data, uint32_t ld, uint32_t lane, uint32_t waveIndex, uint32_t count)
            {
                if constexpr(Count >= 1u && Items * (ItemElems / (Count == 0u ? 1u : Count)) <= MaxWaves)
                {
                    constexpr uint32_t perItem = ItemElems / Count;
                    if(count == Count)
                    {
                        if(waveIndex < Items * perItem)
                            part<Load, Count>(x, waveIndex / perItem, (waveIndex % perItem) * Count, data, ld, lane);
                    }
                    else
                        pieces<Load, Count / 2u>(x, data, ld, lane, waveIndex, count);
                }
            }

            template <bool Load, typename Ptr, typename Reg>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                shared(Reg* x, Ptr* data, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                const uint32_t lane = threadIdx.x & (kWaveSize - 1u);
                if(waveCount > Items && waveCount % Items == 0u && ItemElems % (waveCount / Items) == 0u)
                    pieces<Load, ItemElems / 2u>(x, data, ld, lane, waveIndex, ItemElems / (waveCount / Items));
                else
                {
                    const uint32_t per = (Items + waveCount - 1u) / waveCount;
#pragma unroll
                    for(uint32_t s = 0; s < Items; ++s)
                    {
                        const uint32_t item = waveIndex * per + s;
                        if(s < per && item < Items)
                            part<Load, ItemElems>(x + s * ItemElems, item, 0u, data, ld, lane);
                    }
                }
            }

            ROCWMMA_DEVICE static ROCWMMA_INLINE void load(DataT* x, const DataT* data, uint32_t ld)
            {
                whole<true>(x, data, ld);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void store(DataT* data, const DataT* x, uint32_t ld)
            {
                whole<false>(x, data, ld);
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex)
            {
                shared<true, WaveCount>(x, data, ld, waveIndex);
            }
            template <uint32_t WaveCount>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex)
            {
                shared<false, WaveCount>(x, data, ld, waveIndex);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                loadCoop(DataT* x, const DataT* data, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                shared<true>(x, data, ld, waveIndex, waveCount);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                storeCoop(DataT* data, const DataT* x, uint32_t ld, uint32_t waveIndex, uint32_t waveCount)
            {
                shared<false>(x, data, ld, waveIndex, waveCount);
            }
        };

    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_FRAGMENT_IO_HPP
