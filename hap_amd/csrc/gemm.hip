// MFMA GEMM for gfx950: C = alpha * op(A) * op(B) (+ bias) (act) (+ C), float32 accumulation.
//
// One kernel template serves bf16 (v_mfma_f32_32x32x16_bf16) and float32 (v_mfma_f32_32x32x2_f32) inputs.
// Both operands are staged in LDS as [row][k] with 128 bytes of k per row, so the register fragment of
// either type is one 16-byte LDS read.  Rows are not padded; the eight 16-byte chunks of a row are
// XOR-swizzled with (row ^ row >> 3) & 7, which makes the fragment reads, the row-wise tile stores and the
// transposing tile stores spread over all banks.  An operand whose reduction dimension is the slow one in
// memory (dgrad's weight, both operands of wgrad) is transposed in registers on its way into LDS.
// Ragged M / N / K are handled by guarded edge loads and stores; the interior of every tile runs unguarded
// 16-byte accesses.  Small outputs with a long reduction (wgrad) are split along K over blockIdx.y into
// a caller-provided float32 workspace and summed in split order by a second kernel (deterministic).
//
// The MFMA "A" operand is fed from op(B) rows (n) and the "B" operand from op(A) rows (m): each lane then
// holds 4 consecutive n of one m in its accumulators and the epilogue issues 8/16-byte stores along the
// contiguous dimension of C.
#include "common.h"
#include "tile.h"
#include <vector>
#include <mutex>

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
    int64_t ws_ld;
};

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == HAPMI_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == HAPMI_ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
    return v;
}

template <typename TI, typename TO, int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_kernel(GemmParams p) {
    constexpr int THREADS = WAVES_M * WAVES_N * 64;
    constexpr int EPV = 16 / sizeof(TI);
    constexpr int BK = ROW_BYTES / sizeof(TI);
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KSTEPS = 4;                                     // 32 bytes of k per lane-half pair
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *As = smem;                                              // [2][BM][128 B]
    char *Bs = smem + 2 * A_BYTES;                                // [2][BN][128 B]

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

    const int64_t z1 = blockIdx.z / p.batch2, z2 = blockIdx.z % p.batch2;
    const TI *A = (const TI *)p.A + z1 * p.sA1 + z2 * p.sA2;
    const TI *B = (const TI *)p.B + z1 * p.sB1 + z2 * p.sB2;
    TO *C = (TO *)p.C + z1 * p.sC1 + z2 * p.sC2;

    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const int64_t m_left = p.M - m0, n_left = p.N - n0;

    const int nk_total = (int)((p.K + BK - 1) / BK);
    const int kt0 = (int)blockIdx.y * p.ktiles_per_split;
    const int kt1 = (kt0 + p.ktiles_per_split) < nk_total ? (kt0 + p.ktiles_per_split) : nk_total;
    if (kt0 >= kt1) return;                                       // uniform for the whole block

    const TI *a_base = A_KMAJOR ? A + m0 * p.lda : A + m0;     // element (m0, k=0)
    const TI *b_base = B_KMAJOR ? B + n0 * p.ldb : B + n0;
    const int64_t a_kstep = A_KMAJOR ? (int64_t)BK : (int64_t)BK * p.lda;
    const int64_t b_kstep = B_KMAJOR ? (int64_t)BK : (int64_t)BK * p.ldb;

    TileLoader<TI, BM, THREADS, A_KMAJOR> la;
    TileLoader<TI, BN, THREADS, B_KMAJOR> lb;

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int wm = (wave % WAVES_M) * WTM, wn = (wave / WAVES_M) * WTN;
    const int frow = lane & 31, fh = lane >> 5;

    // byte offset of this lane's fragment for k-step 0 inside a tile; k-step s is at offset ^ (s << 5)
    int a_off[TM], b_off[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = wm + i * 32 + frow;
        a_off[i] = row * ROW_BYTES + ((fh ^ swz(row)) << 4);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int row = wn + j * 32 + frow;
        b_off[j] = row * ROW_BYTES + ((fh ^ swz(row)) << 4);
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
            for (int i = 0; i < TM; ++i) fa[i] = *(const Vec16<TI> *)(as + (a_off[i] ^ (ks << 5)));
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = *(const Vec16<TI> *)(bs + (b_off[j] ^ (ks << 5)));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) Mma<TI>::run(acc[i][j], fb[j], fa[i]);
        }
    };

    // A ragged last k-tile (K not a multiple of the tile depth) is done first, alone, with guarded loads, so
    // that the main loop below only ever sees complete k-tiles and stays free of branches.
    int kt_end = kt1;
    if ((p.K % BK) != 0 && kt1 == nk_total) {
        kt_end = kt1 - 1;
        const int64_t k_left = p.K - (int64_t)kt_end * BK;
        la.load(a_base + (int64_t)kt_end * a_kstep, p.lda, m_left, k_left);
        lb.load(b_base + (int64_t)kt_end * b_kstep, p.ldb, n_left, k_left);
        la.store(As);
        lb.store(Bs);
        __syncthreads();
        compute_tile(As, Bs);
        __syncthreads();
    }

    if (kt0 < kt_end) {
        // complete k-tiles: row-major operands go global -> LDS directly, k-major operands through registers
        // (transposed on the LDS store)
        if (A_KMAJOR) la.init_direct(p.lda, m_left);
        else la.init_offsets(p.lda, m_left);
        if (B_KMAJOR) lb.init_direct(p.ldb, n_left);
        else lb.init_offsets(p.ldb, n_left);
        auto issue_tile = [&](int kt, int buf) {
            if (A_KMAJOR) la.load_direct(a_base + (int64_t)kt * a_kstep, As + buf * A_BYTES);
            else la.load_fast(a_base + (int64_t)kt * a_kstep, p.lda);
            if (B_KMAJOR) lb.load_direct(b_base + (int64_t)kt * b_kstep, Bs + buf * B_BYTES);
            else lb.load_fast(b_base + (int64_t)kt * b_kstep, p.ldb);
        };
        auto commit_tile = [&](int buf) {
            if (!A_KMAJOR) la.store(As + buf * A_BYTES);
            if (!B_KMAJOR) lb.store(Bs + buf * B_BYTES);
            __builtin_amdgcn_s_waitcnt(0x0F70);                   // vmcnt(0): this wave's direct loads have landed
        };
        issue_tile(kt0, 0);
        commit_tile(0);
        __syncthreads();
        for (int kt = kt0; kt < kt_end; ++kt) {
            const int cur = (kt - kt0) & 1;
            if (kt + 1 < kt_end) issue_tile(kt + 1, cur ^ 1);
            compute_tile(As + cur * A_BYTES, Bs + cur * B_BYTES);
            if (kt + 1 < kt_end) commit_tile(cur ^ 1);
            __syncthreads();
        }
    }

    // epilogue: acc[i][j][r] is C[m, n] with m = wm + i*32 + lane%32, n = wn + j*32 + (r/4)*8 + (lane/32)*4 + r%4.
    // Each wave stages one 32-row band of its tile at a time as float32 in a private slice of the (now idle)
    // operand LDS and reads it back row-wise, so that global stores (and the reads of an accumulating C)
    // are whole 128/256-byte row segments instead of 8-byte pieces scattered over 32 rows.
    const bool split = p.splits > 1;
    const bool lead = blockIdx.y == 0;                            // the split that adds the bias
    constexpr int SROW = WTN * 4 + 16;                            // staged row: WTN floats + 16 B (bank spread)
    constexpr int NWAVES = WAVES_M * WAVES_N;
    static_assert(32 * SROW * NWAVES <= 2 * (A_BYTES + B_BYTES), "epilogue staging does not fit the operand LDS");
    char *stage = smem + wave * (32 * SROW);
    constexpr int QPR = WTN / 4;                                  // float4 groups per staged row
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = acc[i][j][q * 4 + e] * p.alpha;
                *(f32x4 *)(stage + (lane & 31) * SROW + (j * 32 + q * 8 + (lane >> 5) * 4) * 4) = o;
            }
        // read back: 32 rows x QPR groups, 64 groups per pass, consecutive lanes along a row
#pragma unroll
        for (int g0 = 0; g0 < 32 * QPR; g0 += 64) {
            const int gidx = g0 + lane;
            if ((32 * QPR) % 64 != 0 && gidx >= 32 * QPR) break;
            const int row = gidx / QPR, qc = gidx % QPR;
            const int64_t m = m0 + wm + i * 32 + row;
            const int64_t n = n0 + wn + qc * 4;
            if (m >= p.M || n >= p.N) continue;
            const f32x4 sv = *(const f32x4 *)(stage + row * SROW + qc * 16);
            float v[4] = {sv[0], sv[1], sv[2], sv[3]};
            const bool full = (n + 4 <= p.N);
            if (p.bias && lead) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (full || n + e < p.N) v[e] += p.bias[n + e];
            }
            if (split) {
                // partial sums of this k-range go to the workspace [split][M][Npad]; a second kernel adds them
                // up in split order and applies activation / accumulation
                float *w = p.ws + ((int64_t)blockIdx.y * p.M + m) * p.ws_ld + n;
                f32x4 o = {v[0], v[1], v[2], v[3]};
                *(f32x4 *)w = o;                                  // ws_ld is a multiple of 4 and >= N rounded up
                continue;
            }
            if (p.act != HAPMI_ACT_NONE) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = apply_act(v[e], p.act);
            }
            TO *dst = C + m * p.ldc + n;
            if (full && ((p.ldc & 3) == 0)) {
                typedef TO out4_t __attribute__((ext_vector_type(4)));
                if (p.accumulate) {
                    const out4_t old = *(const out4_t *)dst;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += (float)old[e];
                }
                out4_t o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (TO)v[e];
                *(out4_t *)dst = o;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (n + e < p.N) {
                        float x = v[e];
                        if (p.accumulate) x += (float)dst[e];
                        dst[e] = (TO)x;
                    }
                }
            }
        }
    }
}

// ---- tile configurations ------------------------------------------------------------------------
struct TileCfg {
    int bm, bn, wm, wn;
};
constexpr TileCfg kCfg[] = {{128, 128, 2, 2}, {256, 256, 2, 4}, {384, 192, 4, 2}, {192, 256, 2, 4}, {256, 192, 4, 2}};
constexpr int kNumCfg = 5;
constexpr int kNumCU = 256;
int g_force_cfg = -1;
int g_force_splits = 0;

// ---- instrumentation: HIP events around every launch --------------------------------------------
struct ProfState {
    std::mutex mu;
    bool on = false;
    std::vector<hipEvent_t> pool;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pending;
    double flops = 0.0;
    int64_t launches = 0;
};
ProfState g_prof;

hipEvent_t prof_event() {
    if (!g_prof.pool.empty()) {
        hipEvent_t e = g_prof.pool.back();
        g_prof.pool.pop_back();
        return e;
    }
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

template <typename TI, typename TO, int BM, int BN, int WM, int WN>
int launch_cfg(const GemmParams &p, int transA, int transB, int64_t batch, hipStream_t st) {
    GemmParams q = p;
    q.tiles_m = (int)hapmi_cdiv(p.M, BM);
    q.tiles_n = (int)hapmi_cdiv(p.N, BN);
    dim3 grid((unsigned)(q.tiles_m * q.tiles_n), (unsigned)q.splits, (unsigned)batch), block(WM * WN * 64);
    const size_t smem = (size_t)2 * (BM + BN) * ROW_BYTES;
#define HAPMI_GEMM_LAUNCH(AK, BK_)                                                                        \
    do {                                                                                                  \
        auto kern = gemm_kernel<TI, TO, BM, BN, WM, WN, AK, BK_>;                                         \
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
    if (!transA && transB) HAPMI_GEMM_LAUNCH(true, true);
    else if (!transA && !transB) HAPMI_GEMM_LAUNCH(true, false);
    else if (transA && !transB) HAPMI_GEMM_LAUNCH(false, false);
    else HAPMI_GEMM_LAUNCH(false, true);
#undef HAPMI_GEMM_LAUNCH
    return HAPMI_OK;
}

// Tile shape and K split are chosen together from a small cost model (units: microseconds):
//   rounds of tiles over the co-resident block slots x (tile FLOPs / per-slot rate + fixed prologue/epilogue)
//   + the split-K reduction traffic.  128x128 tiles run two blocks per CU (512 slots), the 8-wave tiles one.
struct Choice {
    int cfg, splits;
};

Choice choose(int64_t M, int64_t N, int64_t K, int64_t batch, int bk, bool wide, int64_t max_splits, bool row_major_operands) {
    static const int kSplitMenu[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32};
    const int64_t nk = hapmi_cdiv(K, bk);
    Choice best{0, 1};
    double best_t = 1e30;
    for (int c = 0; c < kNumCfg; ++c) {
        if (g_force_cfg >= 0 && g_force_cfg < kNumCfg && c != g_force_cfg && (wide || g_force_cfg == 0)) continue;
        if (c > 0 && !wide) continue;
        if (c == 2 && !row_major_operands && g_force_cfg != 2) continue;   // 384x192 with a transposing loader spills registers
        const int64_t tiles = hapmi_cdiv(M, kCfg[c].bm) * hapmi_cdiv(N, kCfg[c].bn) * batch;
        const double slots = c == 0 ? 2.0 * kNumCU : 1.0 * kNumCU;
        const double rate = c == 0 ? 1.75 : 4.1;                         // TFLOP/s per slot in steady state
        const double fixed = c == 0 ? 2.0 : 3.5;                         // us per tile: first loads + epilogue
        for (int s : kSplitMenu) {
            if (g_force_splits > 0 && s != g_force_splits && !(s == 1 && (max_splits < g_force_splits || batch != 1))) continue;
            if (s > 1 && (s > max_splits || batch != 1 || nk / s < 4)) continue;
            const double tile_us = 2.0 * kCfg[c].bm * kCfg[c].bn * (double)bk * (double)hapmi_cdiv(nk, s) / (rate * 1e6);
            const double rounds = (double)hapmi_cdiv(tiles * s, (int64_t)slots);
            double t = rounds * (tile_us + fixed);
            if (s > 1) t += 2.0 + (double)s * (double)M * (double)N * 8.0 / 3.0e6;   // launch + write/read at ~3 TB/s
            if (t < best_t) {
                best_t = t;
                best = Choice{c, s};
            }
        }
    }
    return best;
}

template <typename TO>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *ws, TO *C, int64_t M, int64_t N, int64_t ws_ld,
                                                          int64_t ldc, int splits, int accumulate, int act) {
    const int64_t groups = ws_ld / 4, total = M * groups;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t m = i / groups, n = (i - m * groups) * 4;
        if (n >= N) continue;
        f32x4 acc = *(const f32x4 *)(ws + m * ws_ld + n);
        for (int s = 1; s < splits; ++s) {
            const f32x4 v = *(const f32x4 *)(ws + ((int64_t)s * M + m) * ws_ld + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += v[e];
        }
        TO *dst = C + m * ldc + n;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e < N) {
                float x = apply_act(acc[e], act);
                if (accumulate) x += (float)dst[e];
                dst[e] = (TO)x;
            }
        }
    }
}

template <typename TI, typename TO>
int launch_typed(GemmParams &p, int transA, int transB, int64_t batch, hipStream_t st, bool wide, void *workspace,
                 int64_t workspace_bytes) {
    const int bk = ROW_BYTES / (int)sizeof(TI);
    const int64_t nk = hapmi_cdiv(p.K, bk);
    p.ws_ld = (p.N + 3) / 4 * 4;
    const int64_t per_split = p.M * p.ws_ld * 4;
    const int64_t max_splits = (workspace && ((uintptr_t)workspace % 16) == 0 && per_split > 0) ? workspace_bytes / per_split : 0;
    const Choice ch = choose(p.M, p.N, p.K, batch, bk, wide && sizeof(TI) == 2, max_splits, !transA && transB);
    const int c = ch.cfg;
    p.splits = ch.splits;
    p.ktiles_per_split = (int)hapmi_cdiv(nk, p.splits);
    p.splits = (int)hapmi_cdiv(nk, p.ktiles_per_split);
    p.ws = (float *)workspace;
    int rc;
    switch (c) {
        case 1: rc = launch_cfg<bf16_t, TO, 256, 256, 2, 4>(p, transA, transB, batch, st); break;
        case 2: rc = launch_cfg<bf16_t, TO, 384, 192, 4, 2>(p, transA, transB, batch, st); break;
        case 3: rc = launch_cfg<bf16_t, TO, 192, 256, 2, 4>(p, transA, transB, batch, st); break;
        case 4: rc = launch_cfg<bf16_t, TO, 256, 192, 4, 2>(p, transA, transB, batch, st); break;
        default: rc = launch_cfg<TI, TO, 128, 128, 2, 2>(p, transA, transB, batch, st);
    }
    if (rc || p.splits <= 1) return rc;
    int64_t gx = hapmi_cdiv(p.M * (p.ws_ld / 4), 256);
    if (gx > 256 * 16) gx = 256 * 16;
    hipLaunchKernelGGL((splitk_reduce_kernel<TO>), dim3((unsigned)gx), dim3(256), 0, st, (const float *)p.ws, (TO *)p.C,
                       p.M, p.N, p.ws_ld, p.ldc, p.splits, p.accumulate, p.act);
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_gemm(const hapmi_gemm_args *a, hapmi_stream_t stream) {
    HAPMI_REQUIRE(a, HAPMI_EINVAL, "gemm: null argument block");
    HAPMI_REQUIRE(hapmi_dtype_ok(a->in_dtype) && hapmi_dtype_ok(a->out_dtype), HAPMI_EINVAL, "gemm: bad dtype");
    HAPMI_REQUIRE(a->M >= 0 && a->N >= 0 && a->K >= 0 && a->batch1 >= 1 && a->batch2 >= 1, HAPMI_EINVAL,
                  "gemm: bad shape M=%lld N=%lld K=%lld", (long long)a->M, (long long)a->N, (long long)a->K);
    if (a->M == 0 || a->N == 0) return HAPMI_OK;
    HAPMI_REQUIRE(a->A && a->B && a->C, HAPMI_EINVAL, "gemm: null pointer");
    HAPMI_REQUIRE(a->act == HAPMI_ACT_NONE || a->act == HAPMI_ACT_RELU || a->act == HAPMI_ACT_GELU, HAPMI_EINVAL,
                  "gemm: unknown activation %d", a->act);
    const int64_t epv = a->in_dtype == HAPMI_F32 ? 4 : 8;
    const int64_t a_cols = a->transA ? a->M : a->K, b_cols = a->transB ? a->K : a->N;
    HAPMI_REQUIRE(a->lda >= a_cols && a->ldb >= b_cols && a->ldc >= a->N, HAPMI_EINVAL,
                  "gemm: leading dimension below the row length (lda=%lld ldb=%lld ldc=%lld)", (long long)a->lda,
                  (long long)a->ldb, (long long)a->ldc);
    HAPMI_REQUIRE(((uintptr_t)a->A % 16) == 0 && ((uintptr_t)a->B % 16) == 0 && a->lda % epv == 0 &&
                      a->ldb % epv == 0 && a->strideA1 % epv == 0 && a->strideA2 % epv == 0 &&
                      a->strideB1 % epv == 0 && a->strideB2 % epv == 0,
                  HAPMI_EALIGN, "gemm: A/B pointers, leading dimensions and batch strides must be 16-byte multiples");
    const int64_t osz = hapmi_elem_size(a->out_dtype);
    HAPMI_REQUIRE(((uintptr_t)a->C % (4 * osz)) == 0 && (a->strideC1 % 4) == 0 && (a->strideC2 % 4) == 0, HAPMI_EALIGN,
                  "gemm: C pointer and batch strides must be multiples of 4 elements");
    const int64_t batch = a->batch1 * a->batch2;
    HAPMI_REQUIRE(batch <= 65535, HAPMI_ELIMIT, "gemm: batch %lld above 65535", (long long)batch);
    HAPMI_REQUIRE(hapmi_cdiv(a->M, 128) * hapmi_cdiv(a->N, 128) < (1ll << 31), HAPMI_ELIMIT, "gemm: too many tiles");

    GemmParams p;
    p.A = a->A; p.B = a->B; p.C = a->C; p.bias = (const float *)a->bias;
    p.M = a->M; p.N = a->N; p.K = a->K;
    p.lda = a->lda; p.ldb = a->ldb; p.ldc = a->ldc;
    p.batch2 = a->batch2;
    p.sA1 = a->strideA1; p.sA2 = a->strideA2; p.sB1 = a->strideB1; p.sB2 = a->strideB2;
    p.sC1 = a->strideC1; p.sC2 = a->strideC2;
    p.alpha = a->alpha; p.accumulate = a->accumulate; p.act = a->act;
    p.tiles_m = p.tiles_n = 0;
    p.splits = 1;
    p.ktiles_per_split = 1;
    p.ws = nullptr;
    p.ws_ld = 0;

    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool prof = false;
    {
        std::lock_guard<std::mutex> lk(g_prof.mu);
        prof = g_prof.on;
        if (prof) {
            e0 = prof_event();
            e1 = prof_event();
            prof = e0 && e1;
        }
    }
    if (prof) (void)hipEventRecord(e0, st);
    int rc;
    if (a->in_dtype == HAPMI_BF16 && a->out_dtype == HAPMI_BF16) rc = launch_typed<bf16_t, bf16_t>(p, a->transA, a->transB, batch, st, true, a->workspace, a->workspace_bytes);
    else if (a->in_dtype == HAPMI_BF16) rc = launch_typed<bf16_t, float>(p, a->transA, a->transB, batch, st, true, a->workspace, a->workspace_bytes);
    else if (a->out_dtype == HAPMI_F32) rc = launch_typed<float, float>(p, a->transA, a->transB, batch, st, false, a->workspace, a->workspace_bytes);
    else rc = launch_typed<float, bf16_t>(p, a->transA, a->transB, batch, st, false, a->workspace, a->workspace_bytes);
    if (prof) {
        (void)hipEventRecord(e1, st);
        std::lock_guard<std::mutex> lk(g_prof.mu);
        g_prof.pending.emplace_back(e0, e1);
        g_prof.flops += 2.0 * (double)a->M * (double)a->N * (double)a->K * (double)batch;
        g_prof.launches += 1;
    }
    if (rc) return rc;
    HAPMI_CHECK_LAUNCH("gemm");
    return HAPMI_OK;
}

extern "C" int hapmi_gemm_tuning(int tile_config, int k_splits) {
    g_force_cfg = tile_config;
    g_force_splits = k_splits;
    return HAPMI_OK;
}

extern "C" int hapmi_prof_gemm_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof.mu);
    g_prof.on = on != 0;
    return HAPMI_OK;
}

extern "C" int hapmi_prof_gemm_collect(double *ms, int64_t *launches, double *flops) {
    std::lock_guard<std::mutex> lk(g_prof.mu);
    double total = 0.0;
    for (auto &pr : g_prof.pending) {
        if (hipEventSynchronize(pr.second) != hipSuccess) return hapmi_set_error(HAPMI_ELAUNCH, "prof: event sync failed");
        float t = 0.f;
        if (hipEventElapsedTime(&t, pr.first, pr.second) != hipSuccess)
            return hapmi_set_error(HAPMI_ELAUNCH, "prof: elapsed time failed");
        total += t;
        g_prof.pool.push_back(pr.first);
        g_prof.pool.push_back(pr.second);
    }
    g_prof.pending.clear();
    if (ms) *ms = total;
    if (launches) *launches = g_prof.launches;
    if (flops) *flops = g_prof.flops;
    g_prof.flops = 0.0;
    g_prof.launches = 0;
    return HAPMI_OK;
}
