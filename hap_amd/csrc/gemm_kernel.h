// MFMA GEMM for gfx950: C = alpha * op(A) * op(B) (+ bias) (act) (+ C), float32 accumulation.
//
// One kernel template serves bf16 (v_mfma_f32_32x32x16_bf16) and float32 (v_mfma_f32_32x32x2_f32) inputs.
// Both operands are staged in LDS as [row][k] with 128 bytes of k per row, so the register fragment of
// either type is one 16-byte LDS read.  Rows are not padded; the eight 16-byte chunks of a row are
// XOR-swizzled with (row ^ row >> 3) & 7, which makes the fragment reads, the row-wise tile stores and the
// transposing tile stores spread over all banks.  An operand whose reduction dimension is the slow one in
// memory (dgrad's weight, both operands of wgrad) is, for bf16, kept in LDS as it lies in memory and
// transposed by the LDS reads that assemble its fragments (TrTile); for float32 it is transposed in
// registers on its way into LDS.
// Ragged M / N / K are handled by guarded edge loads and stores; the interior of every tile runs unguarded
// 16-byte accesses.  Small outputs with a long reduction (wgrad) are split along K over blockIdx.y into
// a caller-provided float32 workspace and summed in split order by a second kernel (deterministic).
//
// The MFMA "A" operand is fed from op(B) rows (n) and the "B" operand from op(A) rows (m): each lane then
// holds 4 consecutive n of one m in its accumulators and the epilogue issues 8/16-byte stores along the
// contiguous dimension of C.
#pragma once
#include "common.h"
#include "dropout.h"
#include "tile.h"
#include <type_traits>

// an operand or result in pieces along one dimension (hapmi_gemm_segments with 32-bit ranges)
struct GemmSegs {
    int n;                                                    // 0 = off
    int begin[HAPMI_GEMM_MAX_SEGMENTS + 1];
    int64_t ld[HAPMI_GEMM_MAX_SEGMENTS];
    const void *base[HAPMI_GEMM_MAX_SEGMENTS];
};

struct GemmParams {
    const void *A, *B;
    void *C;
    const float *bias;
    int64_t M, N, K;
    int64_t lda, ldb, ldc;
    int64_t batch2;
    int64_t sA1, sA2, sB1, sB2, sC1, sC2;
    float alpha;
    int accumulate, act;
    int tiles_m, tiles_n;
    int splits, ktiles_per_split;
    float *ws;                 // split-K workspace [splits][M][ws_ld] (float32)
    float *rowsum;             // optional: rowsum[m] += sum_k op(A)[m, k] (A stored [K, M] only); the blocks write
                               // partial sums to rs_ws, a second kernel adds them up in a fixed order
    float *rs_ws;              // [problem][split][tiles_n][M] partial row sums (float32)
    const void *relu_mask;     // optional: [M][ldc] in C's element type; result elements whose mask is <= 0 become 0
    int64_t ws_ld;
    const void *addend;        // optional (accumulate): the old values are read here instead of from C
    int n_list;                // > 0: problem blockIdx.z takes its pointers from the lists below
    const void *listA[HAPMI_GEMM_MAX_LIST], *listB[HAPMI_GEMM_MAX_LIST];
    void *listC[HAPMI_GEMM_MAX_LIST];
    float *listRS[HAPMI_GEMM_MAX_LIST];
    GemmSegs segA, segB, segC, segM;                          // A along K; B, C and the relu mask along N
    const void *listSegB[HAPMI_GEMM_MAX_LIST][HAPMI_GEMM_MAX_SEGMENTS];   // with pointer lists: the B pieces of problem z
    int a_relu, b_relu;                                       // relu on op(A) / op(B) fragments as they are read
    const int64_t *drop_state;                                // optional: F.dropout behind the activation (RNG state on the device)
    int64_t drop_stream;
    float drop_p;
};
static_assert(sizeof(GemmParams) <= 3072, "the parameter block travels as a kernel argument (4 KiB at most)");

namespace {

template <typename TI> struct Mma;
template <> struct Mma<bf16_t> {
    __device__ __forceinline__ static void run(f32x16 &acc, const Vec16<bf16_t> &a, const Vec16<bf16_t> &b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    __device__ __forceinline__ static void run(f32x16 &acc, const Vec16<float> &a, const Vec16<float> &b) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b.v[i], acc, 0, 0, 0);
    }
};


__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == HAPMI_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == HAPMI_ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
    return v;
}

__device__ __forceinline__ bf16x8 relu_frag(bf16x8 v) {
    // max(x, 0) on bf16 through the signed 16-bit integer order: negative values (sign bit set) become +0
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    return __builtin_bit_cast(bf16x8, __builtin_elementwise_max(__builtin_bit_cast(s16x8, v), zero));
}
__device__ __forceinline__ f32x4 relu_frag(f32x4 v) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = v[e] > 0.f ? v[e] : 0.f;
    return v;
}

// OPMODE bits (compile-time, so that the main loop of every instantiation is free of branches).  1: A is read in
// pieces along K (p.segA; NT layout, three stages, direct loads; a plain A travels as one piece).  2: relu on the
// fragments of op(A).  4: relu on the fragments of op(B) (TN layout: the weight gradient whose B operand is the
// activation that a relu produced).  16: F.dropout behind the
// activation in the epilogue (NT layout: a linear's forward; p.drop_*).  The other kinds of pieces (B, C and the mask along N) only move this block's
// base pointers and leading dimensions, which costs nothing, so they need no instantiation of their own.
template <typename TI, typename TO, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR, int NSTAGES, int OPMODE = 0>
// the four-wave 128 x 128 tile is meant to run two blocks per CU: keep it within 256 registers
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, ((WAVES_M * WAVES_N <= 4 && BM * BN <= 128 * 128) ? 2 : 1)) void gemm_kernel(GemmParams p) {
    constexpr int THREADS = WAVES_M * WAVES_N * 64;
    constexpr int EPV = 16 / sizeof(TI);
    constexpr int BK = ROW_BYTES / sizeof(TI);
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KSTEPS = 4;                                     // 32 bytes of k per lane-half pair
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *As = smem;                                              // [NSTAGES][BM][128 B]
    char *Bs = smem + NSTAGES * A_BYTES;                          // [NSTAGES][BN][128 B]

    // tile mapping: blocks go round-robin over the 8 XCDs; give each XCD a contiguous range of tiles and
    // walk it in columns of 8 m-tiles so that concurrently running tiles share A rows / B columns in L2
    int bid = blockIdx.x;
    const int nblk = gridDim.x;
    if (nblk % 8 == 0) bid = (bid % 8) * (nblk / 8) + bid / 8;
    constexpr int GROUP = 8;
    const int per_group = GROUP * p.tiles_n;
    const int g = bid / per_group;
    const int gm0 = g * GROUP;
    const int gsz = (p.tiles_m - gm0) < GROUP ? (p.tiles_m - gm0) : GROUP;
    const int tm = gm0 + (bid % per_group) % gsz;
    const int tn = (bid % per_group) / gsz;

    const TI *A = (const TI *)p.A;
    const TI *B = (const TI *)p.B;
    TO *C = (TO *)p.C;
    float *rowsum = p.rowsum;
    const TO *rmask = (const TO *)p.relu_mask;                    // laid out like C, batch strides included
    if (p.n_list > 0) {                                           // uniform: scalar loads from the argument block
        const int z = (int)blockIdx.z;
        A = (const TI *)p.listA[z];
        B = (const TI *)p.listB[z];
        C = (TO *)p.listC[z];
        rowsum = p.listRS[z];
    } else if (gridDim.z > 1) {                                   // batch index: at most 65535, 32-bit division
        const int b2 = (int)p.batch2;
        const int64_t z1 = (int)blockIdx.z / b2, z2 = (int)blockIdx.z % b2;
        A += z1 * p.sA1 + z2 * p.sA2;
        B += z1 * p.sB1 + z2 * p.sB2;
        C += z1 * p.sC1 + z2 * p.sC2;
        if (rmask) rmask += z1 * p.sC1 + z2 * p.sC2;
    }

    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t m_left = p.M - m0, n_left = p.N - n0;

    // B, C and the relu mask may exist as pieces along N (no tile straddles a piece): take this block's piece and
    // address it as if it were the whole matrix (base moved back by the piece's first column)
    int64_t ldb = p.ldb, ldc = p.ldc;
    if (p.segB.n > 0) {
        int s = 0;
        while (s + 1 < p.segB.n && n0 >= p.segB.begin[s + 1]) ++s;
        const void *base = p.n_list > 0 ? p.listSegB[(int)blockIdx.z][s] : p.segB.base[s];
        B = (const TI *)base - p.segB.begin[s];
        ldb = p.segB.ld[s];
    }
    if (p.segC.n > 0) {
        int s = 0;
        while (s + 1 < p.segC.n && n0 >= p.segC.begin[s + 1]) ++s;
        C = (TO *)const_cast<void *>(p.segC.base[s]) - p.segC.begin[s];
        ldc = p.segC.ld[s];
        if (p.segM.n > 0) rmask = (const TO *)p.segM.base[s] - p.segC.begin[s];
    }

    // accumulate reads the old values `old_delta` bytes from where the result goes (0: in place)
    const int64_t old_delta = p.addend ? (int64_t)((const char *)p.addend - (const char *)C) : 0;

    const int nk_total = (int)((p.K + BK - 1) / BK);
    const int kt0 = (int)blockIdx.y * p.ktiles_per_split;
    const int kt1 = (kt0 + p.ktiles_per_split) < nk_total ? (kt0 + p.ktiles_per_split) : nk_total;
    if (kt0 >= kt1) return;                                       // uniform for the whole block

    const TI *a_base = A_KMAJOR ? A + m0 * p.lda : A + m0;     // element (m0, k=0)
    const TI *b_base = B_KMAJOR ? B + n0 * ldb : B + n0;
    const int64_t a_kstep = A_KMAJOR ? (int64_t)BK : (int64_t)BK * p.lda;
    const int64_t b_kstep = B_KMAJOR ? (int64_t)BK : (int64_t)BK * ldb;

    // bf16 operands stored [k][row] stay that way in LDS and are transposed by the fragment reads
    constexpr bool A_TR = !A_KMAJOR && sizeof(TI) == 2, B_TR = !B_KMAJOR && sizeof(TI) == 2;
    typedef TrTile<BM, THREADS> TrA;
    typedef TrTile<BN, THREADS> TrB;
    typename std::conditional<A_TR, TrA, TileLoader<TI, BM, THREADS, A_KMAJOR>>::type la;
    typename std::conditional<B_TR, TrB, TileLoader<TI, BN, THREADS, B_KMAJOR>>::type lb;

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = (wave % WAVES_M) * WTM, wn = (wave / WAVES_M) * WTN;
    const int frow = lane & 31, fh = lane >> 5;

    // byte offset of this lane's fragment for k-step 0 inside a tile; k-step s is at offset ^ (s << 5)
    // ([row][k] tiles) or 16 k lines further ([k][row] tiles)
    int a_off[TM], b_off[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = wm + i * 32 + frow;
        if constexpr (A_TR) a_off[i] = TrA::frag_offset(wm + i * 32);
        else a_off[i] = row * ROW_BYTES + ((fh ^ swz(row)) << 4);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int row = wn + j * 32 + frow;
        if constexpr (B_TR) b_off[j] = TrB::frag_offset(wn + j * 32);
        else b_off[j] = row * ROW_BYTES + ((fh ^ swz(row)) << 4);
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    auto compute_tile = [&](const char *as, const char *bs) {
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            Vec16<TI> fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if constexpr (A_TR) fa[i].v = TrA::read_frag(as, a_off[i], ks);
                else fa[i] = *(const Vec16<TI> *)(as + (a_off[i] ^ (ks << 5)));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (B_TR) fb[j].v = TrB::read_frag(bs, b_off[j], ks);
                else fb[j] = *(const Vec16<TI> *)(bs + (b_off[j] ^ (ks << 5)));
            }
            if constexpr ((OPMODE & 2) != 0) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i].v = relu_frag(fa[i].v);
            }
            if constexpr ((OPMODE & 4) != 0) {
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[j].v = relu_frag(fb[j].v);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) Mma<TI>::run(acc[i][j], fb[j], fa[i]);
        }
    };

    // Optional row sums of op(A) (the bias gradient when A is dY of a weight-gradient GEMM), taken from the A
    // tiles as they pass: float32 tiles in registers on their way to LDS (rs_add), bf16 tiles from LDS once
    // they are complete (rs_add_lds).  Every block of a tile row sees the same A tiles, so the k-tiles are
    // dealt round-robin over the tiles_n blocks of the row: each block adds 1/tiles_n of the work instead of
    // one block in tiles_n doing all of it.
    const bool do_rs = !A_KMAJOR && rowsum != nullptr;
    constexpr int RS_N = A_KMAJOR ? 1 : (A_TR ? 8 : TileLoader<TI, BM, THREADS, false>::PASSES_T * EPV);
    float rs[RS_N];
#pragma unroll
    for (int e = 0; e < RS_N; ++e) rs[e] = 0.f;
    auto rs_add = [&]() {
        if constexpr (!A_KMAJOR && !A_TR) {
#pragma unroll
            for (int pp = 0; pp < decltype(la)::PASSES_T; ++pp)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int e = 0; e < EPV; ++e) rs[pp * EPV + e] += la.v[pp * 4 + q].get(e);
        }
    };
    auto rs_add_lds = [&](const char *as) {
        if constexpr (A_TR) TrA::add_row_sums(as, rs);
    };

    // A ragged last k-tile (K not a multiple of the tile depth) is done first, alone, with guarded loads, so
    // that the main loop below only ever sees complete k-tiles and stays free of branches.
    int kt_end = kt1;
    if ((p.K % BK) != 0 && kt1 == nk_total) {
        kt_end = kt1 - 1;
        const int64_t k_left = p.K - (int64_t)kt_end * BK;
        la.load(a_base + (int64_t)kt_end * a_kstep, p.lda, m_left, k_left);
        lb.load(b_base + (int64_t)kt_end * b_kstep, ldb, n_left, k_left);
        if (do_rs && kt_end % p.tiles_n == tn) rs_add();
        la.store(As);
        lb.store(Bs);
        __syncthreads();
        if (do_rs && kt_end % p.tiles_n == tn) rs_add_lds(As);
        compute_tile(As, Bs);
        __syncthreads();
    }

    if (kt0 < kt_end) {
        // complete k-tiles: row-major operands go global -> LDS directly, k-major operands through registers
        // (transposed on the LDS store)
        constexpr bool A_DIRECT = A_KMAJOR || A_TR, B_DIRECT = B_KMAJOR || B_TR;
        if constexpr (A_DIRECT) la.init_direct(p.lda, m_left);
        else la.init_offsets(p.lda, m_left);
        if constexpr (B_DIRECT) lb.init_direct(ldb, n_left);
        else lb.init_offsets(ldb, n_left);
        // A in pieces along K: k-tiles are issued in increasing order, so the piece index only moves forward
        // (the piece's base, end and the loader's row offsets are refreshed only when a k-tile enters the next piece:
        // a few times per launch, not once per k-tile)
        int seg_a = 0, seg_end = 0;
        const TI *seg_base = nullptr;                             // element (m0, k = 0) as if the piece were all of A
        auto issue_tile = [&](int kt, int buf) {
            if constexpr ((OPMODE & 1) != 0) {
                const int k = kt * BK;
                if (k >= seg_end) {
                    while (seg_a + 1 < p.segA.n && k >= p.segA.begin[seg_a + 1]) ++seg_a;
                    const int64_t ld = p.segA.ld[seg_a];
                    la.set_ld((int)ld);
                    seg_base = (const TI *)p.segA.base[seg_a] + m0 * ld - p.segA.begin[seg_a];
                    seg_end = p.segA.begin[seg_a + 1];
                }
                la.load_direct(seg_base + k, As + buf * A_BYTES);
            } else if constexpr (A_DIRECT) la.load_direct(a_base + (int64_t)kt * a_kstep, As + buf * A_BYTES);
            else la.load_fast(a_base + (int64_t)kt * a_kstep, p.lda);
            if constexpr (B_DIRECT) lb.load_direct(b_base + (int64_t)kt * b_kstep, Bs + buf * B_BYTES);
            else lb.load_fast(b_base + (int64_t)kt * b_kstep, ldb);
        };
        auto commit_tile = [&](int buf, int kt) {
            if (do_rs && kt % p.tiles_n == tn) rs_add();
            if constexpr (!A_DIRECT) la.store(As + buf * A_BYTES);
            if constexpr (!B_DIRECT) lb.store(Bs + buf * B_BYTES);
            __builtin_amdgcn_s_waitcnt(0x0F70);                   // vmcnt(0): this wave's direct loads have landed
        };
        if constexpr (NSTAGES == 3) {
            // Three buffers, two k-tiles in flight: a k-tile's loads are issued two iterations before it is
            // multiplied, so their round trip (longer than one iteration of a one-block-per-CU tile) is covered.
            // Both operands go global -> LDS directly (no registers involved); a wave's loads complete in order,
            // so tile kt has landed once at most the loads of tile kt + 1 are outstanding.
            static_assert(A_DIRECT && B_DIRECT, "three stages need direct loads for both operands");
            static_assert((OPMODE & 1) == 0 || (A_KMAJOR && sizeof(TI) == 2), "A in pieces: bf16, stored [M, K]");
            constexpr int LPT = decltype(la)::LOADS_PER_TILE + decltype(lb)::LOADS_PER_TILE;
            static_assert(LPT < 64, "vmcnt holds 6 bits");
            constexpr int WAIT_NEXT = (LPT & 15) | 0x0F70 | ((LPT >> 4) << 14);
            issue_tile(kt0, 0);
            if (kt0 + 1 < kt_end) issue_tile(kt0 + 1, 1);
            int cur = 0;
            for (int kt = kt0; kt < kt_end; ++kt) {
                if (kt + 1 < kt_end) __builtin_amdgcn_s_waitcnt(WAIT_NEXT);
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();                                  // tile kt is complete; everyone is done with tile kt - 1
                const int nxt2 = cur == 0 ? 2 : cur - 1;          // (cur + 2) % 3: the buffer of tile kt - 1
                if (kt + 2 < kt_end) issue_tile(kt + 2, nxt2);
                if (do_rs && kt % p.tiles_n == tn) rs_add_lds(As + cur * A_BYTES);
                compute_tile(As + cur * A_BYTES, Bs + cur * B_BYTES);
                cur = cur == 2 ? 0 : cur + 1;
            }
            __syncthreads();
        } else {
        static_assert((OPMODE & 1) == 0, "A in pieces needs the three-stage loop");
        issue_tile(kt0, 0);
        commit_tile(0, kt0);
        __syncthreads();
        for (int kt = kt0; kt < kt_end; ++kt) {
            const int cur = (kt - kt0) & 1;
            if (kt + 1 < kt_end) issue_tile(kt + 1, cur ^ 1);
            if (do_rs && kt % p.tiles_n == tn) rs_add_lds(As + cur * A_BYTES);
            compute_tile(As + cur * A_BYTES, Bs + cur * B_BYTES);
            if (kt + 1 < kt_end) commit_tile(cur ^ 1, kt + 1);
            __syncthreads();
        }
        }
    }

    if (do_rs) {
        // Every thread's sums go to a slot of their own in the (idle) operand LDS, [group][row] with one group per
        // set of threads that covers all rows once; one thread per row then adds the groups in order and writes the
        // block's partial sum to its slot of the workspace, [problem][split][tile column][M].  No atomics anywhere:
        // the second kernel (rowsum_reduce_kernel) adds the slots of a row in a fixed order, so the result does not
        // depend on the order in which blocks run.
        float *part = (float *)smem;
        constexpr int RS_GROUPS = A_TR ? TrA::KP : BK / 4;
        static_assert(RS_GROUPS * BM * 4 <= NSTAGES * (A_BYTES + B_BYTES), "row-sum staging does not fit the operand LDS");
        if constexpr (A_TR) {
            if ((int)threadIdx.x < TrA::KP * TrA::CPR) {
                float *dst = part + ((int)threadIdx.x / TrA::CPR) * BM + ((int)threadIdx.x % TrA::CPR) * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) dst[e] = rs[e];
            }
        } else if constexpr (!A_KMAJOR) {
            constexpr int RV_ = decltype(la)::RV, BLOCKS_ = decltype(la)::BLOCKS;
#pragma unroll
            for (int pp = 0; pp < decltype(la)::PASSES_T; ++pp) {
                const int blk = threadIdx.x + pp * THREADS;
                if (blk < BLOCKS_) {
                    float *dst = part + (blk / RV_) * BM + (blk % RV_) * EPV;
#pragma unroll
                    for (int e = 0; e < EPV; ++e) dst[e] = rs[pp * EPV + e];
                }
            }
        }
        __syncthreads();
        float *slot = p.rs_ws + (((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * p.tiles_n + tn) * p.M + m0;
        for (int t = threadIdx.x; t < BM; t += THREADS)
            if (t < m_left) {
                float s = 0.f;
#pragma unroll
                for (int g = 0; g < RS_GROUPS; ++g) s += part[g * BM + t];
                slot[t] = s;
            }
        __syncthreads();
    }

    // epilogue: acc[i][j][r] is C[m, n] with m = wm + i*32 + lane%32, n = wn + j*32 + (r/4)*8 + (lane/32)*4 + r%4.
    // Scale, bias and activation are applied to the accumulators in place (one uniform branch per kind, not
    // one per element).  Then each wave stages one 32-row band of its tile at a time in a private slice of the
    // (now idle) operand LDS and reads it back row-wise, so that global stores (and the reads of an
    // accumulating C) are whole 128/256-byte row segments instead of 8-byte pieces scattered over 32 rows.
    // A tile that lies completely inside C (uniform for the block) takes a copy of the store loop without
    // bounds checks: the per-store exec masking of the guarded copy costs more than the stores themselves.
    const bool split = p.splits > 1;
    const bool lead = blockIdx.y == 0;                            // the split that adds the bias
    const bool interior = m_left >= BM && n_left >= BN;
    constexpr int NWAVES = WAVES_M * WAVES_N;

    // The plain bf16 store path below masks the result with relu's derivative (rmask) one 32-row band at a time.  The
    // mask of a band is fetched one band ahead (the first one here, before the accumulators are scaled and staged), so
    // that its trip to memory overlaps the work on the band before instead of stalling every band's stores.
    constexpr int MG16 = WTN / 8, MNG = 32 * MG16 / 64;
    const bool bf16_rows = sizeof(TO) == 2 && !split && !p.accumulate && (ldc & 7) == 0 && ((uintptr_t)C & 15) == 0;
    const bool mask_ahead = bf16_rows && interior && rmask != nullptr;
    bf16x8 mask_v[2][MNG];
    auto fetch_mask = [&](int i) {
        const bf16_t *mband = (const bf16_t *)rmask + (m0 + wm + i * 32) * ldc + n0 + wn;
#pragma unroll
        for (int g = 0; g < MNG; ++g) {
            const int gidx = g * 64 + lane;
            mask_v[i & 1][g] = *(const bf16x8 *)(mband + (gidx / MG16) * (int)ldc + (gidx % MG16) * 8);
        }
    };
    if (mask_ahead) fetch_mask(0);

    if (p.bias && lead) {
        const bool bias_vec = interior && ((uintptr_t)p.bias & 15) == 0;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t n = n0 + wn + j * 32 + q * 8 + (lane >> 5) * 4;
                f32x4 b4;
                if (bias_vec) {
                    b4 = *(const f32x4 *)(p.bias + n);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) b4[e] = n + e < p.N ? p.bias[n + e] : 0.f;
                }
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][q * 4 + e] = acc[i][j][q * 4 + e] * p.alpha + b4[e];
            }
    } else if (p.alpha != 1.0f) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] *= p.alpha;
    }
    if (!split) {
        if (p.act == HAPMI_ACT_RELU) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = acc[i][j][r] > 0.f ? acc[i][j][r] : 0.f;
        } else if (p.act == HAPMI_ACT_GELU) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = apply_act(acc[i][j][r], HAPMI_ACT_GELU);
        }
        if constexpr ((OPMODE & 16) != 0) {
            // F.dropout behind the activation: the decision for C[m][n] is the one the elementwise dropout kernel
            // takes for element m * ldc + n (the host admits one contiguous problem only); registers 4 q + e of a
            // lane are four neighbouring columns, so one hash serves two of them.  For a 2-byte result the value is
            // rounded before it is scaled, as the stored activation would have been.
            const DropKey key = drop_key(p.drop_state[0], p.drop_state[1], p.drop_stream, p.drop_p);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint64_t row_first = (uint64_t)((m0 + wm + i * 32 + (lane & 31)) * ldc + n0 + wn + (lane >> 5) * 4);
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int e = 0; e < 4; e += 2) {
                            const uint32_t bits = drop_pair_bits(key, (row_first + j * 32 + q * 8 + e) >> 1);
                            float lo = acc[i][j][q * 4 + e], hi = acc[i][j][q * 4 + e + 1];
                            if (sizeof(TO) == 2) {
                                lo = (float)(bf16_t)lo;
                                hi = (float)(bf16_t)hi;
                            }
                            acc[i][j][q * 4 + e] = (bits & 0xffffU) >= key.thr ? lo * key.scale : 0.f;
                            acc[i][j][q * 4 + e + 1] = (bits >> 16) >= key.thr ? hi * key.scale : 0.f;
                        }
            }
        }
    }

    // bf16 output that is neither accumulated into nor a split-K partial: the band is staged as bf16 (half the
    // LDS traffic) and leaves in 16-byte stores.  Needs 16-byte alignment of C, its leading dimension and the
    // tile's column origin.
    if (bf16_rows) {
        constexpr int SROWH = WTN * 2 + 16;
        constexpr int G16 = WTN / 8;
        constexpr int NG = 32 * G16 / 64;
        static_assert((32 * G16) % 64 == 0, "wave tile width must be a multiple of 16");
        static_assert(32 * SROWH * NWAVES <= NSTAGES * (A_BYTES + B_BYTES), "epilogue staging does not fit the operand LDS");
        char *stage = smem + wave * (32 * SROWH);
        int soff[NG], goff[NG];                                   // staged / global offsets of this lane's groups
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const int gidx = g * 64 + lane, row = gidx / G16, gc = gidx % G16;
            soff[g] = row * SROWH + gc * 16;
            goff[g] = row * (int)ldc + gc * 8;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    bf16x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = (bf16_t)acc[i][j][q * 4 + e];
                    *(bf16x4 *)(stage + (lane & 31) * SROWH + (j * 32 + q * 8 + (lane >> 5) * 4) * 2) = o;
                }
            bf16_t *band = (bf16_t *)C + (m0 + wm + i * 32) * ldc + n0 + wn;
            const bf16_t *mband = rmask ? (const bf16_t *)rmask + (m0 + wm + i * 32) * ldc + n0 + wn : nullptr;
            if (interior && mband) {
                // the producer of this operand's gradient applied relu itself: its output is the mask
                if (i + 1 < TM) fetch_mask(i + 1);
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    bf16x8 sv = *(const bf16x8 *)(stage + soff[g]);
                    const bf16x8 mv = mask_v[i & 1][g];
#pragma unroll
                    for (int e = 0; e < 8; ++e) sv[e] = (float)mv[e] > 0.f ? sv[e] : (bf16_t)0.f;
                    *(bf16x8 *)(band + goff[g]) = sv;
                }
            } else if (interior) {
#pragma unroll
                for (int g = 0; g < NG; ++g) *(bf16x8 *)(band + goff[g]) = *(const bf16x8 *)(stage + soff[g]);
            } else {
#pragma unroll
                for (int g = 0; g < NG; ++g) {
                    const int gidx = g * 64 + lane, row = gidx / G16, gc = gidx % G16;
                    const int64_t m = m0 + wm + i * 32 + row;
                    const int64_t n = n0 + wn + gc * 8;
                    if (m >= p.M || n >= p.N) continue;
                    bf16x8 sv = *(const bf16x8 *)(stage + soff[g]);
                    bf16_t *dst = band + goff[g];
                    if (mband) {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (n + e < p.N && !((float)mband[goff[g] + e] > 0.f)) sv[e] = (bf16_t)0.f;
                    }
                    if (n + 8 <= p.N) {
                        *(bf16x8 *)dst = sv;
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (n + e < p.N) dst[e] = sv[e];
                    }
                }
            }
        }
        return;
    }

    constexpr int SROW = WTN * 4 + 16;                            // staged row: WTN floats + 16 B (bank spread)
    static_assert(32 * SROW * NWAVES <= NSTAGES * (A_BYTES + B_BYTES), "epilogue staging does not fit the operand LDS");
    char *stage = smem + wave * (32 * SROW);
    constexpr int QPR = WTN / 4;                                  // float4 groups per staged row
    constexpr int NQ = 32 * QPR / 64;
    static_assert((32 * QPR) % 64 == 0, "wave tile width must be a multiple of 8");
    typedef TO out4_t __attribute__((ext_vector_type(4)));
    const bool fast = interior && (ldc & 3) == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = acc[i][j][q * 4 + e];
                *(f32x4 *)(stage + (lane & 31) * SROW + (j * 32 + q * 8 + (lane >> 5) * 4) * 4) = o;
            }
        // read back: 32 rows x QPR groups, 64 groups per pass, consecutive lanes along a row.  Partial sums of a
        // k-range go to the workspace [split][M][ws_ld] (ws_ld a multiple of 4, >= N); a second kernel adds them
        // up in split order and applies activation / accumulation.
        const int64_t mb = m0 + wm + i * 32, nb = n0 + wn;
        if (fast) {
            TO *band = C + mb * ldc + nb;
            float *wband = split ? p.ws + ((int64_t)blockIdx.y * p.M + mb) * p.ws_ld + nb : nullptr;
#pragma unroll
            for (int g = 0; g < NQ; ++g) {
                const int gidx = g * 64 + lane, row = gidx / QPR, qc = gidx % QPR;
                f32x4 v = *(const f32x4 *)(stage + row * SROW + qc * 16);
                if (split) {
                    *(f32x4 *)(wband + row * (int)p.ws_ld + qc * 4) = v;
                    continue;
                }
                TO *dst = band + row * (int)ldc + qc * 4;
                if (rmask) {
                    const out4_t mk = *(const out4_t *)(rmask + (mb + row) * ldc + nb + qc * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (float)mk[e] > 0.f ? v[e] : 0.f;
                }
                if (p.accumulate) {
                    const out4_t old = *(const out4_t *)((const char *)dst + old_delta);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += (float)old[e];
                }
                out4_t o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (TO)v[e];
                *(out4_t *)dst = o;
            }
            continue;
        }
#pragma unroll
        for (int g = 0; g < NQ; ++g) {
            const int gidx = g * 64 + lane;
            const int row = gidx / QPR, qc = gidx % QPR;
            const int64_t m = mb + row;
            const int64_t n = nb + qc * 4;
            if (m >= p.M || n >= p.N) continue;
            const f32x4 v = *(const f32x4 *)(stage + row * SROW + qc * 16);
            if (split) {
                *(f32x4 *)(p.ws + ((int64_t)blockIdx.y * p.M + m) * p.ws_ld + n) = v;
                continue;
            }
            TO *dst = C + m * ldc + n;
            f32x4 vm = v;
            if (rmask) {
                const TO *mk = rmask + m * ldc + n;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < p.N && !((float)mk[e] > 0.f)) vm[e] = 0.f;
            }
            if (n + 4 <= p.N && ((ldc & 3) == 0)) {
                f32x4 x = vm;
                if (p.accumulate) {
                    const out4_t old = *(const out4_t *)((const char *)dst + old_delta);
#pragma unroll
                    for (int e = 0; e < 4; ++e) x[e] += (float)old[e];
                }
                out4_t o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (TO)x[e];
                *(out4_t *)dst = o;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (n + e < p.N) {
                        float x = vm[e];
                        if (p.accumulate) x += (float)*(const TO *)((const char *)(dst + e) + old_delta);
                        dst[e] = (TO)x;
                    }
                }
            }
        }
    }
}

template <typename TI, typename TO, int BM, int BN, int WM, int WN, int NSTAGES = 2>
int launch_cfg(const GemmParams &p, int transA, int transB, int64_t batch, hipStream_t st) {
    GemmParams q = p;
    q.tiles_m = (int)hapmi_cdiv(p.M, BM);
    q.tiles_n = (int)hapmi_cdiv(p.N, BN);
    dim3 grid((unsigned)(q.tiles_m * q.tiles_n), (unsigned)q.splits, (unsigned)batch), block(WM * WN * 64);
    const size_t smem = (size_t)NSTAGES * (BM + BN) * ROW_BYTES;
#define HAPMI_GEMM_LAUNCH(AK, BK_) HAPMI_GEMM_LAUNCH_MODE(AK, BK_, 0)
#define HAPMI_GEMM_LAUNCH_MODE(AK, BK_, MODE)                                                             \
    do {                                                                                                  \
        auto kern = gemm_kernel<TI, TO, BM, BN, WM, WN, AK, BK_, NSTAGES, MODE>;                                 \
        if (smem > 64 * 1024) {                                                                           \
            static bool raised = false;                                                                   \
            if (!raised) {                                                                                \
                if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                        (int)smem) != hipSuccess)                                         \
                    return hapmi_set_error(HAPMI_ELAUNCH, "gemm: cannot raise the LDS limit to %zu", smem); \
                raised = true;                                                                            \
            }                                                                                             \
        }                                                                                                 \
        hipLaunchKernelGGL(kern, grid, block, smem, st, q);                                               \
    } while (0)
    if constexpr (sizeof(TI) == 2) {
        // operand modes (A in pieces along K / relu on an operand): own instantiations of the layouts that use them
        if (p.segA.n > 0) {
            if constexpr (NSTAGES == 3) {
                if (transA || !transB) return hapmi_set_error(HAPMI_EINVAL, "gemm: A_segments / a_relu need transA = 0, transB = 1");
                if (p.a_relu) HAPMI_GEMM_LAUNCH_MODE(true, true, 3);
                else HAPMI_GEMM_LAUNCH_MODE(true, true, 1);
                return HAPMI_OK;
            } else {
                return hapmi_set_error(HAPMI_EINVAL, "gemm: A_segments / a_relu need a three-stage tile configuration");
            }
        }
        if (p.b_relu) {
            if (!transA || transB) return hapmi_set_error(HAPMI_EINVAL, "gemm: b_relu needs transA = 1, transB = 0");
            HAPMI_GEMM_LAUNCH_MODE(false, false, 4);
            return HAPMI_OK;
        }
    }
    if (p.drop_state) {
        if (transA || !transB) return hapmi_set_error(HAPMI_EINVAL, "gemm: dropout in the epilogue needs transA = 0, transB = 1");
        HAPMI_GEMM_LAUNCH_MODE(true, true, 16);
        return HAPMI_OK;
    }
    if (!transA && transB) HAPMI_GEMM_LAUNCH(true, true);
    else if (!transA && !transB) HAPMI_GEMM_LAUNCH(true, false);
    else if (transA && !transB) HAPMI_GEMM_LAUNCH(false, false);
    else HAPMI_GEMM_LAUNCH(false, true);
#undef HAPMI_GEMM_LAUNCH
#undef HAPMI_GEMM_LAUNCH_MODE
    return HAPMI_OK;
}

}  // namespace

// One translation unit per tile configuration (gemm_cfg*.hip) instantiates the kernels of that configuration
// and exports this launcher; gemm.hip picks the configuration and the K split.
#define HAPMI_GEMM_DECLARE_CFG(IDX) \
    int hapmi_gemm_launch_cfg##IDX(const GemmParams &p, int in_dtype, int out_dtype, int transA, int transB, int64_t batch, hipStream_t st)
