// gfx950 data paths between global memory, LDS and MFMA-ready fragments.
//
// Extension of the rocWMMA-style API (no counterpart in the reference, which moves macro
// tiles global -> VGPR -> (shuffle) -> LDS -> VGPR -> (shuffle), see reference
// samples/perf_hgemm.cpp:328-409).  On CDNA4 the same job is done with
//
//   * global_load_lds_dwordx4: each lane copies 16 bytes from global memory straight into
//     LDS (lane i of the issuing wave lands at ldsBase + 16*i) without touching VGPRs;
//   * LDS tiles whose 16-byte chunks are XOR-swizzled so that the ds_read_b128 of an MFMA
//     operand (32 consecutive rows, same K chunk) touches every bank once;
//   * ds_read_b64_tr_b16 for operands stored with the non-K dimension contiguous
//     (column-major A, row-major B): the transposing LDS read returns, to lane i of each
//     16-lane group, the i-th column of a 4 x 16 block whose rows the lanes addressed.
//
// Two LDS tile formats for one pipeline stage of a macro-tile operand of `Dim` rows/columns
// by RowBytes bytes of K (RowBytes = 64: 32 halves or 64 bytes), both filled by whole-wave
// 1 KiB direct copies whose per-lane source offset does not depend on the copy index:
//
//   KMajorTile   -- one operand row per LDS row (row-major A / col-major B).
//   DimMajorTile -- one K index per LDS row of Dim elements (col-major A / row-major B),
//                   16-bit elements; DimMajorTile8 is its 8-bit twin (ds_read_b64_tr_b8).
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

        // The same copy marked non-temporal: for data that is read once (it should not displace
        // operand panels other workgroups are about to re-read from the caches).
        ROCWMMA_DEVICE ROCWMMA_INLINE void asyncCopy16Streaming(void* ldsBase, const void* src)
        {
            __builtin_amdgcn_global_load_lds((GlobalPtr)src, (LdsPtr)ldsBase, 16, 0, 2 /* nt */);
        }

        // The same copy with buffer addressing: source address = resource base + waveOffset
        // (scalar) + laneOffset (one VGPR).  Nothing but scalar arithmetic is needed per copy,
        // which keeps the vector ALU and the VGPR file out of the copy path.
        using BufferRsrc = __amdgpu_buffer_rsrc_t;

        ROCWMMA_DEVICE ROCWMMA_INLINE BufferRsrc makeSource(const void* base)
        {
            // raw buffer, no stride, 2 GiB window from `base`, 32-bit data format
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7FFFFFFF, 0x00020000);
        }

        // The same with the window ending at `end` (one past the last readable byte; at most 2 GiB
        // from `base`): copies of bytes beyond it read nothing and store zeros.
        ROCWMMA_DEVICE ROCWMMA_INLINE BufferRsrc makeSource(const void* base, const void* end)
        {
            const ptrdiff_t left  = static_cast<const char*>(end) - static_cast<const char*>(base);
            const int       bytes = left <= 0 ? 0 : (left > 0x7FFFFFFF ? 0x7FFFFFFF : static_cast<int>(left));
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
        }

        ROCWMMA_DEVICE ROCWMMA_INLINE void asyncCopy16(void* ldsBase, BufferRsrc src, uint32_t laneOffset, uint32_t waveOffset)
        {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                src, (LdsPtr)ldsBase, 16, static_cast<int>(laneOffset), static_cast<int>(waveOffset), 0, 0);
        }

        // The buffer-addressed copy marked non-temporal (data that is read once).
        ROCWMMA_DEVICE ROCWMMA_INLINE void
            asyncCopy16Streaming(void* ldsBase, BufferRsrc src, uint32_t laneOffset, uint32_t waveOffset)
        {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                src, (LdsPtr)ldsBase, 16, static_cast<int>(laneOffset), static_cast<int>(waveOffset), 0, 2 /* nt */);
        }

        // s_waitcnt with "at most MaxLoads vector-memory operations still in flight" and all of
        // this wave's LDS reads returned.  Direct-to-LDS copies complete in issue order, so
        // leaving the newest MaxLoads outstanding means every older copy has landed.
        template <uint32_t MaxLoads>
        ROCWMMA_DEVICE ROCWMMA_INLINE void waitCopiesAndReads()
        {
            static_assert(MaxLoads < 64u, "vmcnt is a 6-bit counter");
            // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
            constexpr uint32_t imm = (MaxLoads & 15u) | (7u << 4) | (0u << 8) | ((MaxLoads >> 4) << 14);
            __builtin_amdgcn_s_waitcnt(imm);
        }

        // Waits until every LDS read this wave has issued has returned (vector-memory copies may
        // stay in flight).  Needed before the registers filled by DimMajorTile::readBlock32 are
        // used: those reads are issued outside the compiler's dependency tracking.
        ROCWMMA_DEVICE ROCWMMA_INLINE void waitReads()
        {
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0), vmcnt / expcnt untouched
        }

        // Ties registers that inline-assembly LDS reads (DimMajorTile::readBlock16 / readBlock32) have
        // written to this point of the program: call it right after the wait that covers those reads
        // and before the values are used.  The reads are outside the compiler's dependency
        // tracking; an empty asm statement that takes each register as an in-out operand makes every
        // later use depend on a statement that cannot be moved in front of the wait.
        template <typename T>
        ROCWMMA_DEVICE ROCWMMA_INLINE void pinRegisters(T& value)
        {
            static_assert(sizeof(T) % 4u == 0u, "whole 32-bit registers");
            typedef uint32_t word_t __attribute__((may_alias));
            word_t* words = reinterpret_cast<word_t*>(&value);
#pragma unroll
            for(uint32_t i = 0; i < sizeof(T) / 4u; ++i)
                asm volatile("" : "+v"(words[i]));
        }

        // Bare workgroup barrier (no implied memory waits: pair it with waitCopiesAndReads).
        ROCWMMA_DEVICE ROCWMMA_INLINE void barrier()
        {
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }

        // ---------------------------------------------------------------------------------
        // K-major stage: Dim rows of 64 bytes (four 16-byte chunks).  Chunk c of row r lives at
        // chunk position c ^ swz(r).
        //
        // Bank behaviour of ds_read_b128, found with the bank-conflict counter and two active lanes
        // at a time: the LDS serves 16 lanes per cycle (256 bytes, every bank once), and the 16 lanes
        // served together are those with the same lane bit 5 and the same parity of lane bits 2, 3, 4
        // (lane 0 goes with 1-3, 12-15 and 20-27).  Both operand patterns must put such a group on 16
        // distinct 16-byte bank groups:
        //   32-wide blocks: row = lane % 32, chunk = lane / 32     -> any bijective swz of row bits 2..3
        //   16-wide blocks: row = lane % 16, chunk = lane / 16     -> lane bit 4 is a chunk bit; needs
        //                   swz(0), swz(3), swz(1)^1, swz(2)^1 distinct and the same with 0/3 and 1/2
        //                   swapped (argument = row bits 2..3)
        // swz = 0, 2, 3, 1 for rows 0-3, 4-7, 8-11, 12-15 satisfies both.
        // ---------------------------------------------------------------------------------
        //
        // With RowBytes = 128 a row is one whole 128-byte line of the operand (eight chunks), so a
        // copy instruction requests eight full lines instead of sixteen half lines.  Two rows then
        // span the 256 bytes the banks cover, and the 16 lanes served together must differ in
        // (row parity, chunk position): swz = row bits 1..3 does that for both readers (the eight
        // even rows of a 16-row group get eight different XOR masks; of the two K chunks a group
        // touches, one goes with masks {0,1,6,7} and the other, differing in bit 0, with {2,3,4,5}).
        //
        // Pairs = true (128-byte rows only) is the variant for 16-wide blocks that take 32 bytes of K per
        // lane (v_mfma_f32_16x16x128_f8f6f4): lane l reads chunks 2 (l / 16) and 2 (l / 16) + 1 of row
        // l % 16 in two instructions.  Lane bit 4 is then chunk bit 1 and is tied to row bits 2, 3 by the
        // parity rule above, so the XOR mask must leave chunk bit 1 free of row bit 3 or of row bit 2:
        // swz = (row bit 3, row bit 3, row bit 1) puts each of the two reads on 16 distinct bank groups
        // (checked by enumeration; the mask of the general variant gives two-way conflicts here).
        template <uint32_t Dim, uint32_t RowBytes = 64u, bool Pairs = false>
        struct KMajorTile
        {
            static_assert(RowBytes == 64u || RowBytes == 128u, "stage rows of 64 or 128 bytes");
            static_assert(!Pairs || RowBytes == 128u, "the pair reader works on 128-byte rows");
            static constexpr uint32_t rowBytes    = RowBytes;
            static constexpr uint32_t chunks      = RowBytes / 16u;
            static constexpr uint32_t rowsPerCopy = 1024u / rowBytes; // 16 or 8
            static constexpr uint32_t bytes       = Dim * rowBytes;
            static constexpr uint32_t copies      = bytes / 1024u; // whole-wave copies per stage

            ROCWMMA_HOST_DEVICE static constexpr uint32_t swz(uint32_t row)
            {
                if constexpr(RowBytes == 64u)
                    return (0x78u >> ((row >> 1) & 6u)) & 3u; // 0, 2, 3, 1 for rows 0-3, 4-7, 8-11, 12-15
                else if constexpr(Pairs)
                    return (((row >> 3) & 1u) * 6u) | ((row >> 1) & 1u);
                else
                    return (row >> 1) & 7u;
            }
            ROCWMMA_HOST_DEVICE static constexpr uint32_t offset(uint32_t row, uint32_t chunk)
            {
                return row * rowBytes + ((chunk ^ swz(row)) << 4);
            }
            // Source byte offset of `lane` inside a copy issued by wave `wave`, relative to the copy's
            // first row at the stage's first K byte: lane i owns LDS position (row i / chunks, chunk
            // position i % chunks).  swz looks at row bits below 4 only; copy c of a wave starts at row
            // (c * waves + wave) * rowsPerCopy, and waves * rowsPerCopy is a multiple of 16 for every
            // wave pool used, so the copy index does not matter, only the wave.
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t laneSourceOffset(uint32_t lane, uint32_t wave, uint32_t ldBytes)
            {
                const uint32_t row = lane / chunks;
                return row * ldBytes + (((lane % chunks) ^ swz(wave * rowsPerCopy + row)) << 4);
            }
            // Source byte offset of copy `copy` (wave uniform)
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t copySourceOffset(uint32_t copy, uint32_t ldBytes)
            {
                return copy * rowsPerCopy * ldBytes;
            }
            // Bytes between consecutive stages along K in global memory
            ROCWMMA_DEVICE static ROCWMMA_INLINE size_t stageStep(uint32_t /*ldBytes*/)
            {
                return rowBytes;
            }

            // Operand of one 32-wide MFMA block: rows [row0, row0+32), K step `ks` of the stage.
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

            // Operand of one 16-wide MFMA block with 16 bytes of K per lane (16x16x32 f16 / bf16,
            // 16x16x64 i8): rows [row0, row0+16), 64 bytes of K (K step `ks` of the stage); lane l
            // holds row l % 16, chunk 4 ks + l / 16.  A quarter-wave reads 16 rows at one chunk index:
            // 16 distinct bank groups by the choice of swz.
            template <uint32_t KPackBytes>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock16(void* regs, const char* ldsTile, uint32_t row0, uint32_t ks, uint32_t lane)
            {
                static_assert(KPackBytes == 16u || (KPackBytes == 32u && Pairs),
                              "16-wide blocks take 16 bytes of K per lane, or 32 from the pair variant");
                constexpr uint32_t perLane = KPackBytes / 16u;
                const uint32_t     row     = row0 + (lane & 15u);
#pragma unroll
                for(uint32_t j = 0; j < perLane; ++j)
                    reinterpret_cast<detail::u32x4*>(regs)[j] = *reinterpret_cast<const detail::u32x4*>(
                        ldsTile + offset(row, (ks * 4u + (lane >> 4)) * perLane + j));
            }
        };

        // ---------------------------------------------------------------------------------
        // Dim-major stage (16-bit elements): 32 LDS rows (one per K index) of Dim elements.
        // Rows are cut into 32-byte segments (16 elements); segment s of K row k lives at
        // segment position s ^ swz(k).  A half-wave touches, in one transposing read, either four
        // K rows of two neighbouring segments (32-wide blocks) or K rows k..k+3 and k+8..k+11 of
        // one segment (16-wide blocks): swz puts both patterns on eight distinct 32-byte positions.
        // ---------------------------------------------------------------------------------
        template <uint32_t Dim, uint32_t KRows = 32u>
        struct DimMajorTile
        {
            static_assert(Dim % 128u == 0u, "tile rows must hold at least eight 32-byte segments");
            static_assert(KRows == 32u || KRows == 64u, "stages of 32 or 64 K rows");
            static constexpr uint32_t kRows       = KRows;
            static constexpr uint32_t rowBytes    = Dim * 2u;
            static constexpr uint32_t bytes       = kRows * rowBytes;
            static constexpr uint32_t copies      = bytes / 1024u;
            static constexpr uint32_t slotsPerRow = rowBytes / 16u; // 16-byte copy slots per K row
            static_assert(slotsPerRow <= 64u ? (64u % slotsPerRow == 0u) : (slotsPerRow % 64u == 0u),
                          "a copy must cover whole K rows or an even part of one");
            static constexpr uint32_t rowsPerCopy = slotsPerRow <= 64u ? 64u / slotsPerRow : 1u;
            static_assert(slotsPerRow <= 64u, "tiles wider than 512 elements are not supported");

            ROCWMMA_HOST_DEVICE static constexpr uint32_t swz(uint32_t k)
            {
                return ((k & 3u) << 1) | ((k >> 3) & 1u);
            }
            ROCWMMA_HOST_DEVICE static constexpr uint32_t offset(uint32_t k, uint32_t seg)
            {
                return k * rowBytes + ((seg ^ swz(k)) << 5);
            }
            // Source byte offset of `lane` inside a copy issued by wave `wave` of a pool whose
            // size times rowsPerCopy is a multiple of 16 (so k & 15 is the same for all its copies).
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t laneSourceOffset(uint32_t lane, uint32_t wave, uint32_t ldBytes)
            {
                const uint32_t kInCopy = lane / slotsPerRow;
                const uint32_t pos     = lane % slotsPerRow;
                const uint32_t k       = wave * rowsPerCopy + kInCopy; // only k & 15 matters
                const uint32_t seg     = (pos >> 1) ^ swz(k);
                return kInCopy * ldBytes + (seg << 5) + ((pos & 1u) << 4);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t copySourceOffset(uint32_t copy, uint32_t ldBytes)
            {
                return copy * rowsPerCopy * ldBytes;
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE size_t stageStep(uint32_t ldBytes)
            {
                return static_cast<size_t>(kRows) * ldBytes;
            }

            // Operand of one 32-wide MFMA block with 8 K values per lane (v_mfma_*_32x32x16):
            // lane l ends up with dim = dim0 + l % 32 and k = ks*16 + (l/32)*8 + 0..7.
            //
            // The transposing reads are written as inline assembly on purpose: as compiler
            // intrinsics they are assumed to alias every direct-to-LDS copy in flight and get a
            // full vmcnt(0) wait in front of them, which serialises the copy pipeline.  The price
            // is that the caller must call lds::waitReads() (or another wait that covers LDS reads)
            // and then lds::pinRegisters() on the destination before the registers are consumed.
            template <uint32_t KPackBytes = 16u>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock32(void* regs, const char* ldsTile, uint32_t dim0, uint32_t ks, uint32_t lane)
            {
                static_assert(KPackBytes == 16u, "transposing reads feed the 8-halves-per-lane MFMA shapes");
                typedef short s16x4 __attribute__((ext_vector_type(4)));
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)ldsTile));
                const uint32_t group   = lane >> 4; // 16-lane group
                const uint32_t s     = lane & 15u; // source index inside the group
                const uint32_t seg   = (dim0 >> 4) + (group & 1u);
                const uint32_t kBase = ks * 16u + (group >> 1) * 8u + (s >> 2);
                const uint32_t inSeg = (s & 3u) << 3; // 4 elements = 8 bytes per source lane
#pragma unroll
                for(uint32_t kk = 0; kk < 2u; ++kk)
                {
                    const uint32_t k    = kBase + kk * 4u;
                    const uint32_t addr = ldsBase + offset(k, seg) + inSeg;
                    s16x4          v;
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                    reinterpret_cast<s16x4*>(regs)[kk] = v;
                }
            }

            // Operand of one 16-wide MFMA block with 8 K values per lane (v_mfma_*_16x16x32):
            // lane l ends up with dim = dim0 + l % 16 and k = 32 ks + (l/16)*8 + 0..7 (32 K rows
            // per step).  Same remarks as for readBlock32.
            template <uint32_t KPackBytes = 16u>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock16(void* regs, const char* ldsTile, uint32_t dim0, uint32_t ks, uint32_t lane)
            {
                static_assert(KPackBytes == 16u, "transposing reads feed the 8-halves-per-lane MFMA shapes");
                typedef short s16x4 __attribute__((ext_vector_type(4)));
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)ldsTile));
                const uint32_t group   = lane >> 4;
                const uint32_t s       = lane & 15u;
                const uint32_t seg     = dim0 >> 4;
                const uint32_t kBase   = ks * 32u + group * 8u + (s >> 2);
                const uint32_t inSeg   = (s & 3u) << 3;
#pragma unroll
                for(uint32_t kk = 0; kk < 2u; ++kk)
                {
                    const uint32_t k    = kBase + kk * 4u;
                    const uint32_t addr = ldsBase + offset(k, seg) + inSeg;
                    s16x4          v;
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                    reinterpret_cast<s16x4*>(regs)[kk] = v;
                }
            }
        };


        // ---------------------------------------------------------------------------------
        // Dim-major stage of 8-bit elements (int8, fp8): KRows LDS rows (one per K index) of Dim bytes,
        // cut into 16-byte segments; segment s of K row k lives at segment position s ^ swz(k).
        //
        // ds_read_b64_tr_b8, found by reading a table of byte ids back: within each group of 16 lanes,
        // result lane t receives, as its byte j (0..7), byte t % 8 of the 8 bytes that lane
        // 2 j + t / 8 of the group addressed.  With lanes 2 j and 2 j + 1 pointing at the two halves of
        // 16 consecutive elements of K row k0 + j, lane t ends up with element t of the K rows
        // k0 .. k0 + 7: a transposed 8 x 16 block, eight consecutive K values per lane.
        //
        // A group's read touches 8 K rows at one segment; rows are Dim bytes apart (a multiple of 128), so
        // swz must spread the rows of one read, and of the two lane groups served together (K rows 16
        // apart for 16-wide blocks), over distinct 16-byte bank groups: the low K bits, and bit 4 above them.
        // ---------------------------------------------------------------------------------
        template <uint32_t Dim, uint32_t KRows>
        struct DimMajorTile8
        {
            static_assert(Dim == 128u || Dim == 256u, "tile rows of 128 or 256 bytes");
            static_assert(KRows == 64u || KRows == 128u, "stages of 64 or 128 K rows");
            static constexpr uint32_t kRows       = KRows;
            static constexpr uint32_t rowBytes    = Dim;
            static constexpr uint32_t bytes       = kRows * rowBytes;
            static constexpr uint32_t copies      = bytes / 1024u;
            static constexpr uint32_t slotsPerRow = rowBytes / 16u; // 8 or 16 segments
            static constexpr uint32_t rowsPerCopy = 64u / slotsPerRow; // 8 or 4 K rows per whole-wave copy

            // (128-byte rows: two K rows share a 256-byte bank window, so K bit 0 already separates them)
            ROCWMMA_HOST_DEVICE static constexpr uint32_t swz(uint32_t k)
            {
                return Dim == 128u ? (((k >> 1) & 3u) | (((k >> 4) & 1u) << 2)) : ((k & 7u) | (((k >> 4) & 1u) << 3));
            }
            ROCWMMA_HOST_DEVICE static constexpr uint32_t offset(uint32_t k, uint32_t seg)
            {
                return k * rowBytes + ((seg ^ swz(k)) << 4);
            }
            // Source byte offset of `lane` inside a copy issued by wave `wave` of a pool whose size times
            // rowsPerCopy is a multiple of 32 (so k % 32 is the same for all of a wave's copies).
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t laneSourceOffset(uint32_t lane, uint32_t wave, uint32_t ldBytes)
            {
                const uint32_t kInCopy = lane / slotsPerRow;
                const uint32_t pos     = lane % slotsPerRow;
                const uint32_t k       = wave * rowsPerCopy + kInCopy; // only k % 32 matters
                return kInCopy * ldBytes + ((pos ^ swz(k)) << 4);
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE uint32_t copySourceOffset(uint32_t copy, uint32_t ldBytes)
            {
                return copy * rowsPerCopy * ldBytes;
            }
            ROCWMMA_DEVICE static ROCWMMA_INLINE size_t stageStep(uint32_t ldBytes)
            {
                return static_cast<size_t>(kRows) * ldBytes;
            }

            // One transposing read: the lane's group reads K rows k0 .. k0 + 7 of the 16 elements that
            // start at dim16 (a multiple of 16); the lane receives element dim16 + lane % 16.
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                read8(uint32_t (&out)[2], uint32_t ldsBase, uint32_t k0, uint32_t dim16, uint32_t lane)
            {
                typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
                const uint32_t s    = lane & 15u;
                const uint32_t k    = k0 + (s >> 1);
                const uint32_t addr = ldsBase + offset(k, dim16 >> 4) + ((s & 1u) << 3);
                u32x2_t        v;
                asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(v) : "v"(addr) : "memory");
                out[0] = v[0];
                out[1] = v[1];
            }

            // Operand of one 16-wide MFMA block with 16 K values per lane (v_mfma_i32_16x16x64_i8):
            // lane l ends up with dim = dim0 + l % 16 and k = 64 ks + (l / 16) * 16 + 0..15.
            // As for the 16-bit tile, the caller waits for the reads and pins the registers before use.
            template <uint32_t KPackBytes>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock16(void* regs, const char* ldsTile, uint32_t dim0, uint32_t ks, uint32_t lane)
            {
                static_assert(KPackBytes == 16u, "16-wide blocks of 8-bit types take 16 bytes of K per lane");
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)ldsTile));
                const uint32_t kBase   = ks * 64u + (lane >> 4) * 16u;
#pragma unroll
                for(uint32_t kk = 0; kk < 2u; ++kk)
                    read8(reinterpret_cast<uint32_t(*)[2]>(regs)[kk], ldsBase, kBase + 8u * kk, dim0, lane);
            }

            // Operand of one 32-wide MFMA block: lane l ends up with dim = dim0 + l % 32 and
            // k = KPackBytes * (2 ks + l / 32) + 0 .. KPackBytes - 1 (16 for v_mfma_i32_32x32x32_i8, 32 for
            // v_mfma_f32_32x32x64_f8f6f4).
            template <uint32_t KPackBytes>
            ROCWMMA_DEVICE static ROCWMMA_INLINE void
                readBlock32(void* regs, const char* ldsTile, uint32_t dim0, uint32_t ks, uint32_t lane)
            {
                const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsPtr)ldsTile));
                const uint32_t kBase   = KPackBytes * (2u * ks + (lane >> 5));
                const uint32_t dim16   = dim0 + (lane & 16u);
#pragma unroll
                for(uint32_t kk = 0; kk < KPackBytes / 8u; ++kk)
                    read8(reinterpret_cast<uint32_t(*)[2]>(regs)[kk], ldsBase, kBase + 8u * kk, dim16, lane);
            }
        };

    } // namespace lds
} // namespace rocwmma

#endif // ROCWMMA_LDS_HPP
