// LDS operand tiles shared by the GEMM and attention kernels: [row][k] with 128 bytes of k per row, the eight
// 16-byte chunks of a row XOR-swizzled with (row ^ row >> 3) & 7, and the loaders that fill them from global
// memory (row-major operands directly, k-major operands through a 4 x EPV register transpose).
#pragma once
#include "common.h"

constexpr int ROW_BYTES = 128;                       // k bytes per LDS row
__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// Loads one operand tile [ROWS][BK] (row = m or n index, k = reduction index) from global memory into
// registers and stores it into the swizzled LDS tile.  KMAJOR: memory is [row][k] (k contiguous);
// otherwise memory is [k][row] (row contiguous) and 4(k) x EPV(row) register blocks are transposed.
template <typename TI, int ROWS, int THREADS, bool KMAJOR> struct TileLoader {
    static constexpr int EPV = 16 / sizeof(TI);
    static constexpr int BK = ROW_BYTES / sizeof(TI);
    static constexpr int KV = 8;                                  // 16-byte chunks per row
    static constexpr int ROWS_PER_PASS = THREADS / KV;
    static constexpr int PASSES_K = ROWS / ROWS_PER_PASS;
    static constexpr int RV = ROWS / EPV;                         // row-vectors per k line
    static constexpr int BLOCKS = (BK / 4) * RV;
    static constexpr int PASSES_T = (BLOCKS + THREADS - 1) / THREADS;
    static constexpr int NV = KMAJOR ? PASSES_K : PASSES_T * 4;
    static_assert(!KMAJOR || (ROWS % ROWS_PER_PASS == 0 && PASSES_K >= 1), "tile does not divide over the block");

    Vec16<TI> v[NV];

    // ---- branch-free path for k-tiles that lie completely inside K -------------------------------------
    // Rows beyond rows_left are clamped to the last valid row / row-vector: they are loaded (in bounds) and
    // multiplied, but the epilogue never stores them.  A row-vector that straddles rows_left stays inside
    // the operand's leading dimension, which is a multiple of the vector width.
    static constexpr int NOFF = KMAJOR ? PASSES_K : PASSES_T;
    int off[NOFF];                                                // element offsets from the tile's base

    __device__ __forceinline__ void init_offsets(int64_t ld, int64_t rows_left) {
        const int t = threadIdx.x;
        const int last = (int)(rows_left < ROWS ? rows_left : ROWS) - 1;
        if (KMAJOR) {
            const int kv = t % KV, r0 = t / KV;
#pragma unroll
            for (int p = 0; p < PASSES_K; ++p) {
                int row = r0 + p * ROWS_PER_PASS;
                row = row < last ? row : last;
                off[p] = row * (int)ld + kv * EPV;
            }
        } else {
            const int last_rr = (last / EPV) * EPV;
#pragma unroll
            for (int p = 0; p < PASSES_T; ++p) {
                int blk = t + p * THREADS;
                blk = blk < BLOCKS ? blk : BLOCKS - 1;            // idle threads repeat the last block (never stored)
                const int rv = blk % RV, kg = blk / RV;
                int rr = rv * EPV;
                rr = rr < last_rr ? rr : last_rr;
                off[p] = kg * 4 * (int)ld + rr;
            }
        }
    }

    // ---- direct global -> LDS path (row-major operands only) ---------------------------------------------
    // One global_load_lds_dwordx4 per wave fills 1024 contiguous LDS bytes = 8 tile rows; lane l lands in row
    // l / 8, physical chunk l % 8, so it fetches the logical chunk (l % 8) ^ swz(row) of that row.
    static constexpr int NWAVES = THREADS / 64;
    static constexpr int PASSES_D = ROWS / (8 * NWAVES);
    int doff[KMAJOR ? (PASSES_D > 0 ? PASSES_D : 1) : 1];

    __device__ __forceinline__ void init_direct(int64_t ld, int64_t rows_left) {
        static_assert(!KMAJOR || ROWS % (8 * NWAVES) == 0, "direct loads need ROWS to be a multiple of 8 * waves");
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int last = (int)(rows_left < ROWS ? rows_left : ROWS) - 1;
#pragma unroll
        for (int p = 0; p < PASSES_D; ++p) {
            const int row = (p * NWAVES + wave) * 8 + (lane >> 3);
            const int chunk = (lane & 7) ^ swz(row);
            doff[p] = (row < last ? row : last) * (int)ld + chunk * EPV;
        }
    }

    __device__ __forceinline__ void load_direct(const TI *base, char *lds) const {
        // Issued as inline assembly on purpose: for the builtin the compiler cannot tell which LDS reads alias
        // the in-flight transfer and waits for vmcnt(0) before every ds_read, which serialises the prefetch
        // with the MFMA loop.  The caller waits for vmcnt(0) itself before the barrier that publishes the tile.
        typedef __attribute__((address_space(3))) char lds_char;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int p = 0; p < PASSES_D; ++p) {
            const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_char *)(lds + (p * NWAVES + wave) * 8 * ROW_BYTES);
            const TI *src = base + doff[p];
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :
                         : "s"(lds_addr), "v"(src)
                         : "memory");
        }
    }

    __device__ __forceinline__ void load_fast(const TI *base, int64_t ld) {
        if (KMAJOR) {
#pragma unroll
            for (int p = 0; p < PASSES_K; ++p) v[p] = *(const Vec16<TI> *)(base + off[p]);
        } else {
#pragma unroll
            for (int p = 0; p < PASSES_T; ++p)
#pragma unroll
                for (int q = 0; q < 4; ++q) v[p * 4 + q] = *(const Vec16<TI> *)(base + off[p] + q * (int)ld);
        }
    }

    __device__ __forceinline__ static Vec16<TI> guarded(const TI *p, int64_t n_valid) {
        Vec16<TI> r;
#pragma unroll
        for (int e = 0; e < EPV; ++e) r.set(e, (e < n_valid) ? ld_f(p, e) : 0.f);
        return r;
    }

    // base: pointer to element (row0, k0) of the operand; rows_left / k_left: valid extent from there
    __device__ __forceinline__ void load(const TI *base, int64_t ld, int64_t rows_left, int64_t k_left) {
        const int t = threadIdx.x;
        if (KMAJOR) {
            const int kv = t % KV, r0 = t / KV;
#pragma unroll
            for (int p = 0; p < PASSES_K; ++p) {
                const int row = r0 + p * ROWS_PER_PASS;
                const int64_t kk = (int64_t)kv * EPV;
                const TI *src = base + (int64_t)row * ld + kk;
                if (row < rows_left && kk + EPV <= k_left) v[p] = *(const Vec16<TI> *)src;
                else if (row < rows_left && kk < k_left) v[p] = guarded(src, k_left - kk);
                else v[p] = guarded(src, 0);
            }
        } else {
#pragma unroll
            for (int p = 0; p < PASSES_T; ++p) {
                const int blk = t + p * THREADS;
                if (BLOCKS % THREADS != 0 && blk >= BLOCKS) break;
                const int rv = blk % RV, kg = blk / RV;
                const int64_t rr = (int64_t)rv * EPV;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int64_t kk = (int64_t)kg * 4 + q;
                    const TI *src = base + kk * ld + rr;
                    if (kk < k_left && rr + EPV <= rows_left) v[p * 4 + q] = *(const Vec16<TI> *)src;
                    else if (kk < k_left && rr < rows_left) v[p * 4 + q] = guarded(src, rows_left - rr);
                    else v[p * 4 + q] = guarded(src, 0);
                }
            }
        }
    }

    __device__ __forceinline__ void store(char *lds) const {
        const int t = threadIdx.x;
        if (KMAJOR) {
            const int kv = t % KV, r0 = t / KV;
#pragma unroll
            for (int p = 0; p < PASSES_K; ++p) {
                const int row = r0 + p * ROWS_PER_PASS;
                *(Vec16<TI> *)(lds + row * ROW_BYTES + ((kv ^ swz(row)) << 4)) = v[p];
            }
        } else {
            typedef TI quad_t __attribute__((ext_vector_type(4)));
            constexpr int QB = 4 * sizeof(TI);                    // bytes of 4 consecutive k: 8 (bf16) or 16 (f32)
#pragma unroll
            for (int p = 0; p < PASSES_T; ++p) {
                const int blk = t + p * THREADS;
                if (BLOCKS % THREADS != 0 && blk >= BLOCKS) break;
                const int rv = blk % RV, kg = blk / RV;
                const int kbyte = kg * QB;                        // logical byte offset inside the row
                const int chunk = kbyte >> 4, within = kbyte & 15;
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    quad_t q4;
#pragma unroll
                    for (int q = 0; q < 4; ++q) q4[q] = v[p * 4 + q].v[e];
                    const int row = rv * EPV + e;
                    *(quad_t *)(lds + row * ROW_BYTES + ((chunk ^ swz(row)) << 4) + within) = q4;
                }
            }
        }
    }
};

