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
    static constexpr int LOADS_PER_TILE = PASSES_D;               // direct-load instructions per wave and tile
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
            drow[p] = row < last ? row : last;
            dchunk[p] = chunk * EPV;
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

    // another leading dimension for the rows of init_direct (an operand that exists in pieces with different
    // leading dimensions): the clamped row and the chunk of every pass are kept for that
    int drow[KMAJOR ? (PASSES_D > 0 ? PASSES_D : 1) : 1], dchunk[KMAJOR ? (PASSES_D > 0 ? PASSES_D : 1) : 1];
    __device__ __forceinline__ void set_ld(int ld) {
#pragma unroll
        for (int p = 0; p < PASSES_D; ++p) doff[p] = drow[p] * ld + dchunk[p];
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

// A bf16 operand whose reduction dimension is the slow one in memory ([k][row], rows contiguous) kept in LDS
// the way it lies in memory: [64 k][ROWS] with the 16-byte chunks (8 rows) of a k line XOR-swizzled.  It goes
// global -> LDS directly (no registers, no transposing stores); the MFMA fragment (8 consecutive k of one row
// per lane) is assembled by two transposing LDS reads (ds_read_b64_tr_b16).  Within each group of 16 lanes
// that instruction hands lane j the elements D[4e + j/4][j%4], e = 0..3, of the 16 x 4 matrix D whose row i
// is the 8 bytes at lane i's address: with lane i pointing at k line i/4, rows 4*(i%4).., lane j receives 4
// consecutive k of row j.  The swizzle makes the 4 k lines x 64 bytes that a half wave touches in one read
// fall into different banks: a line is a multiple of 256 bytes -> chunk ^= 4*(k%4); 384-byte lines (ROWS
// 192) already alternate between bank halves -> chunk ^= 4*((k/2)%2).
template <int ROWS, int THREADS> struct TrTile {
    static constexpr int BK = 64;
    static constexpr int CPR = ROWS / 8;                          // 16-byte chunks per k line
    static constexpr int LINE = ROWS * 2;                         // bytes per k line
    static constexpr int CHUNKS = BK * CPR;
    static constexpr int PASSES = CHUNKS / THREADS;
    static constexpr int LOADS_PER_TILE = PASSES;                 // direct-load instructions per wave and tile
    static_assert(ROWS % 64 == 0 && CHUNKS % THREADS == 0, "tile does not divide over the block");
    static_assert(CPR % 16 == 0 || CPR % 16 == 8, "no bank swizzle for this line length");
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s lds_v4s;

    __device__ __forceinline__ static int sw(int k) { return CPR % 16 == 0 ? ((k & 3) << 2) : (((k >> 1) & 1) << 2); }

    int doff[PASSES];
    bf16x8 v[PASSES];                                             // ragged last k-tile only

    // rows beyond rows_left are clamped to the last valid chunk (loaded in bounds, never stored by the epilogue)
    __device__ __forceinline__ void init_direct(int64_t ld, int64_t rows_left) {
        const int last_c = ((int)(rows_left < ROWS ? rows_left : ROWS) - 1) >> 3;
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int q = p * THREADS + threadIdx.x, k = q / CPR;
            int c = (q % CPR) ^ sw(k);
            c = c < last_c ? c : last_c;
            doff[p] = k * (int)ld + c * 8;
        }
    }

    __device__ __forceinline__ void load_direct(const bf16_t *base, char *lds) const {
        typedef __attribute__((address_space(3))) char lds_char;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_char *)(lds + (p * (THREADS / 64) + wave) * 1024);
            const bf16_t *src = base + doff[p];
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :
                         : "s"(lds_addr), "v"(src)
                         : "memory");
        }
    }

    // guarded path for a k-tile that ends inside K
    __device__ __forceinline__ void load(const bf16_t *base, int64_t ld, int64_t rows_left, int64_t k_left) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int q = p * THREADS + threadIdx.x, k = q / CPR;
            const int r0 = ((q % CPR) ^ sw(k)) * 8;
            const bf16_t *src = base + (int64_t)k * ld + r0;
            if (k < k_left && r0 + 8 <= rows_left) {
                v[p] = *(const bf16x8 *)src;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[p][e] = (k < k_left && r0 + e < rows_left) ? src[e] : (bf16_t)0.f;
            }
        }
    }
    __device__ __forceinline__ void store(char *lds) const {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) *(bf16x8 *)(lds + (p * THREADS + threadIdx.x) * 16) = v[p];
    }

    // byte offset of this lane's first transposing read for the 32-row fragment starting at row r0 (k-step 0)
    __device__ __forceinline__ static int frag_offset(int r0) {
        const int lane = threadIdx.x & 63, i16 = lane & 15;
        const int k = 8 * (lane >> 5) + (i16 >> 2);
        const int row = r0 + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
        return k * LINE + (((row >> 3) ^ sw(k)) << 4) + ((row & 7) << 1);
    }
    __device__ __forceinline__ static bf16x8 read_frag(const char *tile, int off, int ks) {
        union { v4s h[2]; bf16x8 v; } u;
        u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(tile + off + ks * 16 * LINE));
        u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(tile + off + ks * 16 * LINE + 4 * LINE));
        return u.v;
    }

    // sums over k of the tile's rows: thread t < KP * CPR owns the 8 rows of chunk t % CPR on k lines t / CPR + i * KP
    static constexpr int KP = THREADS / CPR;
    static constexpr int RS_PASSES = (BK + KP - 1) / KP;
    __device__ __forceinline__ static void add_row_sums(const char *tile, float (&rs)[8]) {
        const int t = threadIdx.x;
        if (t >= KP * CPR) return;
        const int c = t % CPR;
#pragma unroll
        for (int i = 0; i < RS_PASSES; ++i) {
            const int k = t / CPR + i * KP;
            if (k < BK) {
                const bf16x8 x = *(const bf16x8 *)(tile + k * LINE + ((c ^ sw(k)) << 4));
#pragma unroll
                for (int e = 0; e < 8; ++e) rs[e] += (float)x[e];
            }
        }
    }
};
