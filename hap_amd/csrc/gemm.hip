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
#include "gemm_kernel.h"
#include <string.h>
#include <vector>
#include <mutex>
#include <map>
#include <tuple>

HAPMI_GEMM_DECLARE_CFG(0);
HAPMI_GEMM_DECLARE_CFG(1);
HAPMI_GEMM_DECLARE_CFG(2);
HAPMI_GEMM_DECLARE_CFG(3);
HAPMI_GEMM_DECLARE_CFG(4);
HAPMI_GEMM_DECLARE_CFG(5);
HAPMI_GEMM_DECLARE_CFG(6);
HAPMI_GEMM_DECLARE_CFG(7);
HAPMI_GEMM_DECLARE_CFG(8);
HAPMI_GEMM_DECLARE_CFG(9);
HAPMI_GEMM_DECLARE_CFG(10);
HAPMI_GEMM_DECLARE_CFG(11);

namespace {

// ---- tile configurations ------------------------------------------------------------------------
struct TileCfg {
    int bm, bn, wm, wn;
};
constexpr TileCfg kCfg[] = {{128, 128, 2, 2}, {256, 256, 2, 4}, {384, 192, 4, 2}, {192, 256, 2, 4}, {256, 192, 4, 2},
                             {256, 128, 4, 2}, {128, 256, 2, 4}, {192, 128, 2, 4}, {256, 128, 2, 2}, {128, 192, 4, 2},
                             {64, 64, 2, 2}, {64, 128, 2, 2}};
constexpr int kNumCfg = 12;
constexpr bool is_f32_cfg(int c) { return c == 10 || c == 11; }   // small tiles for float32 operands only
constexpr int kNumCU = 256;
int g_force_cfg = -1;
int g_force_splits = 0;

// ---- plan table: (M, N, K, batch, transA, transB, in, out) -> (configuration, splits) ------------
typedef std::tuple<int64_t, int64_t, int64_t, int64_t, int, int, int, int> PlanKey;
std::map<PlanKey, std::pair<int, int>> g_plans;
std::mutex g_plans_mu;

// ---- instrumentation: HIP events around every launch --------------------------------------------
struct ProfState {
    std::mutex mu;
    bool on = false;
    std::vector<hipEvent_t> pool;
    struct Bracket { hipEvent_t e0, e1, e2; };
    std::vector<Bracket> pending;
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

// Tile shape and K split are chosen together from a small cost model (units: microseconds):
//   rounds of tiles over the co-resident block slots x (tile FLOPs / per-slot rate + fixed prologue/epilogue)
//   + the split-K reduction traffic.  128x128 tiles run two blocks per CU (512 slots), the 8-wave tiles one.
struct Choice {
    int cfg, splits;
};

// Which tile configurations a call may use: 0 serves every type; 1..9 bf16 operands of calls that allow the large
// tiles; 10, 11 float32 operands; 12 only when forced (a measurement build).
// A call with operands in pieces narrows the choice further (SegNeeds): A in pieces along K runs on the three-stage
// configurations only, and the tile's N extent must divide every piece boundary of B / C.
struct SegNeeds {
    bool three_stage = false;
    int64_t n_align = 0;                       // 0: no constraint; else every piece boundary along N is a multiple of it
};
constexpr bool kThreeStage[] = {false, false, false, false, false, true, true, true, true, true, false, false};

bool cfg_eligible(int c, bool bf16_in, bool wide, bool row_major_operands, bool forced, const SegNeeds &need = SegNeeds()) {
    if (need.three_stage && !kThreeStage[c]) return false;
    if (need.n_align > 0 && need.n_align % kCfg[c].bn != 0) return false;
    if (c == 0) return true;
    if (is_f32_cfg(c)) return !bf16_in;
    if (!bf16_in || !wide) return false;
    if (c == 2 && !row_major_operands && !forced) return false;          // 384x192 with a transposing loader spills registers
    return true;
}

Choice choose(int64_t M, int64_t N, int64_t K, int64_t batch, int bk, bool bf16_in, bool wide, int64_t max_splits,
              bool row_major_operands, const SegNeeds &need) {
    static const int kSplitMenu[] = {1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16, 24, 32};
    const int64_t nk = hapmi_cdiv(K, bk);
    Choice best{-1, 1};
    double best_t = 1e30;
    const bool forced = g_force_cfg >= 0 && g_force_cfg < kNumCfg && cfg_eligible(g_force_cfg, bf16_in, wide, row_major_operands, true, need);
    for (int c = 0; c < kNumCfg; ++c) {
        if (forced ? c != g_force_cfg : !cfg_eligible(c, bf16_in, wide, row_major_operands, false, need)) continue;
        const int64_t tiles = hapmi_cdiv(M, kCfg[c].bm) * hapmi_cdiv(N, kCfg[c].bn) * batch;
        // co-resident blocks per CU, TFLOP/s per block slot in steady state, us per tile for first loads + epilogue
        double per_cu, rate, fixed;
        if (bf16_in) {
            per_cu = c == 0 ? 2.0 : 1.0;
            rate = c == 0 ? 1.75 : 4.1;
            fixed = c == 0 ? 2.0 : 3.5;
        } else {                                                         // float32 MFMA: 0.61 TFLOP/s per CU at best
            per_cu = c == 0 ? 2.0 : 4.0;
            rate = 0.5 / per_cu;
            fixed = 2.0;
        }
        const double slots = per_cu * kNumCU;
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
    // nothing matched the forced split: the 128 x 128 tile without a split serves every call it is eligible for
    if (best.cfg < 0 && cfg_eligible(0, bf16_in, wide, row_major_operands, false, need)) best = Choice{0, 1};
    return best;
}

template <typename TO>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *ws, TO *C, int64_t M, int64_t N, int64_t ws_ld,
                                                          int64_t ldc, int splits, int accumulate, int act,
                                                          const TO *relu_mask, const TO *addend) {
    // the partial sums of one output group are independent loads: they are issued eight at a time and added in
    // split order afterwards (the order fixes the float32 result)
    constexpr int U = 8;
    const int64_t groups = ws_ld / 4, total = M * groups;
    const int64_t split_stride = M * ws_ld;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t m = i / groups, n = (i - m * groups) * 4;
        if (n >= N) continue;
        const float *src = ws + m * ws_ld + n;
        f32x4 acc = *(const f32x4 *)src;
        for (int s0 = 1; s0 < splits; s0 += U) {
            f32x4 v[U];
#pragma unroll
            for (int j = 0; j < U; ++j)
                if (s0 + j < splits) v[j] = *(const f32x4 *)(src + (int64_t)(s0 + j) * split_stride);
#pragma unroll
            for (int j = 0; j < U; ++j)
                if (s0 + j < splits) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += v[j][e];
                }
        }
        TO *dst = C + m * ldc + n;
        const TO *prev = addend ? addend + m * ldc + n : dst;     // what an accumulating call adds to
        if (n + 4 <= N && (ldc & 3) == 0 && !relu_mask) {
            typedef TO out4_t __attribute__((ext_vector_type(4)));
            out4_t o;
            if (accumulate) {
                const out4_t old = *(const out4_t *)prev;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (TO)(apply_act(acc[e], act) + (float)old[e]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (TO)apply_act(acc[e], act);
            }
            *(out4_t *)dst = o;
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e < N) {
                float x = apply_act(acc[e], act);
                if (relu_mask && !((float)relu_mask[m * ldc + n + e] > 0.f)) x = 0.f;
                if (accumulate) x += (float)prev[e];
                dst[e] = (TO)x;
            }
        }
    }
}

// The second half of a_rowsum: out[z][m] += the partial row sums of problem z, row m, added in the order (split, tile
// column).  One thread per row and problem; the order fixes the float32 result.
struct RowsumOuts {
    float *out[HAPMI_GEMM_MAX_LIST];
};
__global__ __launch_bounds__(256) void rowsum_reduce_kernel(const float *ws, RowsumOuts outs, int64_t M, int parts) {
    const int z = blockIdx.y;
    float *out = outs.out[z];
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (!out || m >= M) return;
    const float *src = ws + (int64_t)z * parts * M + m;
    float s = 0.f;
    for (int q = 0; q < parts; ++q) s += src[(int64_t)q * M];
    out[m] += s;
}

template <typename TI, typename TO>
int launch_typed(GemmParams &p, int transA, int transB, int64_t batch, hipStream_t st, bool wide, void *workspace,
                 int64_t workspace_bytes, const SegNeeds &need) {
    const int bk = ROW_BYTES / (int)sizeof(TI);
    const int64_t nk = hapmi_cdiv(p.K, bk);
    p.ws_ld = (p.N + 3) / 4 * 4;
    const int64_t per_split = p.M * p.ws_ld * 4;
    bool want_rs = p.rowsum != nullptr;
    for (int z = 0; z < p.n_list; ++z) want_rs = want_rs || p.listRS[z] != nullptr;
    // with row sums the workspace is shared: split-K partials in its first half, partial row sums in the second
    const int64_t rs_off = want_rs ? (workspace_bytes / 2) / 16 * 16 : 0;
    const int64_t split_bytes = want_rs ? rs_off : workspace_bytes;
    if (want_rs && (!workspace || ((uintptr_t)workspace % 16) != 0))
        return hapmi_set_error(HAPMI_EINVAL, "gemm: a_rowsum needs a 16-byte aligned workspace for its partial sums");
    const bool segmented = p.segA.n > 0 || p.segB.n > 0 || p.segC.n > 0;
    // dropout in the epilogue is applied by the GEMM kernel itself, so the reduction is not split then
    const int64_t max_splits = (!segmented && !p.drop_state && workspace && ((uintptr_t)workspace % 16) == 0 && per_split > 0) ? split_bytes / per_split : 0;
    Choice ch = choose(p.M, p.N, p.K, batch, bk, sizeof(TI) == 2, wide, max_splits, !transA && transB, need);
    if (ch.cfg < 0)
        return hapmi_set_error(HAPMI_EINVAL, "gemm: no tile configuration fits the pieces of the operands (boundaries along N "
                               "must be multiples of a tile's N extent: 64, 128, 192 or 256)");
    if (g_force_cfg < 0 && g_force_splits <= 0) {
        std::lock_guard<std::mutex> lk(g_plans_mu);
        auto it = g_plans.find(PlanKey(p.M, p.N, p.K, batch, (int)(transA != 0), (int)(transB != 0), sizeof(TI) == 2 ? HAPMI_BF16 : HAPMI_F32,
                                       sizeof(TO) == 2 ? HAPMI_BF16 : HAPMI_F32));
        if (it != g_plans.end()) {
            const int pc = it->second.first, ps = it->second.second;
            const bool cfg_ok = pc >= 0 && pc < kNumCfg && cfg_eligible(pc, sizeof(TI) == 2, wide, !transA && transB, true, need);
            const bool split_ok = ps == 1 || (ps > 1 && ps <= max_splits && batch == 1 && nk / ps >= 1);
            if (cfg_ok && split_ok) ch = Choice{pc, ps};
        }
    }
    const int c = ch.cfg;
    p.splits = ch.splits;
    p.ktiles_per_split = (int)hapmi_cdiv(nk, p.splits);
    p.splits = (int)hapmi_cdiv(nk, p.ktiles_per_split);
    p.ws = (float *)workspace;
    int rs_parts = 0;
    p.rs_ws = nullptr;
    if (want_rs) {
        rs_parts = p.splits * (int)hapmi_cdiv(p.N, kCfg[c].bn);
        const int64_t need = batch * rs_parts * p.M * 4;
        if (need > workspace_bytes - rs_off)
            return hapmi_set_error(HAPMI_ELIMIT, "gemm: a_rowsum needs %lld bytes in the second half of the workspace, %lld given",
                                   (long long)need, (long long)(workspace_bytes - rs_off));
        p.rs_ws = (float *)((char *)workspace + rs_off);
    }
    const int in_dtype = sizeof(TI) == 2 ? HAPMI_BF16 : HAPMI_F32, out_dtype = sizeof(TO) == 2 ? HAPMI_BF16 : HAPMI_F32;
    int rc;
    switch (c) {
        case 1: rc = hapmi_gemm_launch_cfg1(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 2: rc = hapmi_gemm_launch_cfg2(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 3: rc = hapmi_gemm_launch_cfg3(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 4: rc = hapmi_gemm_launch_cfg4(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 5: rc = hapmi_gemm_launch_cfg5(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 6: rc = hapmi_gemm_launch_cfg6(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 7: rc = hapmi_gemm_launch_cfg7(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 8: rc = hapmi_gemm_launch_cfg8(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 9: rc = hapmi_gemm_launch_cfg9(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 10: rc = hapmi_gemm_launch_cfg10(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        case 11: rc = hapmi_gemm_launch_cfg11(p, in_dtype, out_dtype, transA, transB, batch, st); break;
        default: rc = hapmi_gemm_launch_cfg0(p, in_dtype, out_dtype, transA, transB, batch, st);
    }
    if (rc) return rc;
    if (want_rs) {
        RowsumOuts outs;
        for (int z = 0; z < HAPMI_GEMM_MAX_LIST; ++z) outs.out[z] = p.n_list > 0 ? p.listRS[z] : (z == 0 ? p.rowsum : nullptr);
        hipLaunchKernelGGL(rowsum_reduce_kernel, dim3((unsigned)hapmi_cdiv(p.M, 256), (unsigned)batch), dim3(256), 0, st,
                           (const float *)p.rs_ws, outs, p.M, rs_parts);
    }
    if (p.splits <= 1) return HAPMI_OK;
    int64_t gx = hapmi_cdiv(p.M * (p.ws_ld / 4), 256);
    if (gx > 256 * 16) gx = 256 * 16;
    hipLaunchKernelGGL((splitk_reduce_kernel<TO>), dim3((unsigned)gx), dim3(256), 0, st, (const float *)p.ws, (TO *)p.C,
                       p.M, p.N, p.ws_ld, p.ldc, p.splits, p.accumulate, p.act, (const TO *)p.relu_mask,
                       (const TO *)p.addend);
    return HAPMI_OK;
}

}  // namespace

namespace {
int64_t gcd64(int64_t a, int64_t b) {
    while (b) {
        const int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// copy a description of pieces into the kernel's parameter block after checking it
int fill_segments(GemmSegs &g, const hapmi_gemm_segments *s, int64_t extent, int64_t align, int64_t epv, bool need_base,
                  const char *what) {
    g.n = 0;
    if (!s) return HAPMI_OK;
    HAPMI_REQUIRE(s->n >= 1 && s->n <= HAPMI_GEMM_MAX_SEGMENTS, HAPMI_ELIMIT, "gemm: %s holds 1..%d pieces", what, HAPMI_GEMM_MAX_SEGMENTS);
    HAPMI_REQUIRE(s->begin[0] == 0 && s->begin[s->n] == extent && extent < (1ll << 31), HAPMI_EINVAL,
                  "gemm: %s must cover [0, %lld)", what, (long long)extent);
    for (int i = 0; i < s->n; ++i) {
        const int64_t len = s->begin[i + 1] - s->begin[i];
        HAPMI_REQUIRE(len > 0 && s->begin[i] % align == 0, HAPMI_EINVAL, "gemm: %s: piece %d starts at %lld (not a multiple of %lld) or is empty",
                      what, i, (long long)s->begin[i], (long long)align);
        HAPMI_REQUIRE(s->ld[i] >= len && s->ld[i] % epv == 0, HAPMI_EALIGN, "gemm: %s: leading dimension of piece %d", what, i);
        HAPMI_REQUIRE(!need_base || (s->base[i] && ((uintptr_t)s->base[i] % 16) == 0), HAPMI_EALIGN, "gemm: %s: base of piece %d", what, i);
        g.begin[i] = (int)s->begin[i];
        g.ld[i] = s->ld[i];
        g.base[i] = s->base[i];
    }
    g.begin[s->n] = (int)extent;
    g.n = s->n;
    return HAPMI_OK;
}
}  // namespace

extern "C" int hapmi_gemm(const hapmi_gemm_args *a, hapmi_stream_t stream) {
    HAPMI_REQUIRE(a, HAPMI_EINVAL, "gemm: null argument block");
    HAPMI_REQUIRE(hapmi_dtype_ok(a->in_dtype) && hapmi_dtype_ok(a->out_dtype), HAPMI_EINVAL, "gemm: bad dtype");
    HAPMI_REQUIRE(a->M >= 0 && a->N >= 0 && a->K >= 0 && a->batch1 >= 1 && a->batch2 >= 1, HAPMI_EINVAL,
                  "gemm: bad shape M=%lld N=%lld K=%lld", (long long)a->M, (long long)a->N, (long long)a->K);
    if (a->M == 0 || a->N == 0) return HAPMI_OK;
    const bool lists = a->A_list || a->B_list || a->C_list || a->a_rowsum_list;
    if (lists) {
        HAPMI_REQUIRE(a->A_list && a->B_list && a->C_list, HAPMI_EINVAL, "gemm: A_list, B_list and C_list go together");
        HAPMI_REQUIRE(a->batch1 <= HAPMI_GEMM_MAX_LIST && a->batch2 == 1, HAPMI_ELIMIT,
                      "gemm: pointer lists hold at most %d problems (batch2 = 1)", HAPMI_GEMM_MAX_LIST);
        HAPMI_REQUIRE(!a->A && !a->B && !a->C && !a->a_rowsum && !a->c_relu_mask && !a->c_addend, HAPMI_EINVAL,
                      "gemm: A, B, C, a_rowsum, c_relu_mask and c_addend must be NULL next to pointer lists");
        HAPMI_REQUIRE(!a->a_rowsum_list || a->transA, HAPMI_EINVAL, "gemm: a_rowsum_list needs transA = 1");
        for (int64_t z = 0; z < a->batch1; ++z) {
            HAPMI_REQUIRE(a->A_list[z] && a->B_list[z] && a->C_list[z], HAPMI_EINVAL, "gemm: null pointer in a list");
            HAPMI_REQUIRE(((uintptr_t)a->A_list[z] % 16) == 0 && ((uintptr_t)a->B_list[z] % 16) == 0 &&
                              ((uintptr_t)a->C_list[z] % (4 * hapmi_elem_size(a->out_dtype))) == 0,
                          HAPMI_EALIGN, "gemm: misaligned pointer in a list");
        }
    } else {
        HAPMI_REQUIRE((a->A || a->A_segments) && (a->B || a->B_segments) && (a->C || a->C_segments), HAPMI_EINVAL, "gemm: null pointer");
    }
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
    p.rowsum = a->a_rowsum;
    HAPMI_REQUIRE(!a->a_rowsum || (a->transA && a->batch1 * a->batch2 == 1), HAPMI_EINVAL,
                  "gemm: a_rowsum needs transA = 1 (A stored [K, M]) and a single problem");
    p.addend = a->c_addend;
    HAPMI_REQUIRE(!a->c_addend || (a->accumulate && a->batch1 * a->batch2 == 1 &&
                                   ((uintptr_t)a->c_addend % (4 * osz)) == 0),
                  HAPMI_EINVAL, "gemm: c_addend needs accumulate = 1, a single problem and C's alignment");
    p.n_list = lists ? (int)a->batch1 : 0;
    for (int z = 0; z < HAPMI_GEMM_MAX_LIST; ++z) {
        const bool on = z < p.n_list;
        p.listA[z] = on ? a->A_list[z] : nullptr;
        p.listB[z] = on ? a->B_list[z] : nullptr;
        p.listC[z] = on ? a->C_list[z] : nullptr;
        p.listRS[z] = on && a->a_rowsum_list ? a->a_rowsum_list[z] : nullptr;
    }
    p.relu_mask = a->c_relu_mask;
    HAPMI_REQUIRE(!a->c_relu_mask || (!lists && ((uintptr_t)a->c_relu_mask % 16) == 0), HAPMI_EINVAL,
                  "gemm: c_relu_mask needs a 16-byte aligned pointer and no pointer lists");
    p.drop_state = a->drop_state;
    p.drop_stream = a->drop_stream_id;
    p.drop_p = a->drop_p;
    if (a->drop_state) {
        HAPMI_REQUIRE(!lists && batch == 1 && !a->transA && a->transB && !a->accumulate && a->ldc == a->N && (a->N % 2) == 0 && !a->C_segments &&
                          !a->A_segments && !a->B_segments && !a->c_mask_segments && !a->B_segments_list && !a->a_relu && !a->b_relu &&
                          ((uintptr_t)a->drop_state % 8) == 0 && a->drop_p >= 0.f && a->drop_p <= 1.f,
                      HAPMI_EINVAL, "gemm: dropout in the epilogue takes one contiguous problem (transA = 0, transB = 1, ldc = N, N even), no accumulate, "
                      "no pieces, no relu on an operand, and a probability in [0, 1]");
    }

    // operands / result in pieces
    SegNeeds need;
    memset(p.listSegB, 0, sizeof(p.listSegB));
    p.a_relu = a->a_relu != 0;
    p.b_relu = a->b_relu != 0;
    const bool any_seg = a->A_segments || a->B_segments || a->C_segments || a->c_mask_segments || a->B_segments_list;
    if (any_seg || p.a_relu || p.b_relu)
        HAPMI_REQUIRE(a->in_dtype == HAPMI_BF16 && a->batch2 == 1, HAPMI_EINVAL, "gemm: pieces and operand relu take bf16 operands");
    int rc_seg = fill_segments(p.segA, a->A_segments, a->K, 64, 8, true, "A_segments");
    if (rc_seg) return rc_seg;
    if (p.segA.n > 0 || p.a_relu) {
        HAPMI_REQUIRE(!a->transA && a->transB && batch == 1 && a->K % 64 == 0 && !a->a_rowsum, HAPMI_EINVAL,
                      "gemm: A_segments / a_relu need transA = 0, transB = 1, one problem and K a multiple of 64");
        need.three_stage = true;
        if (p.segA.n == 0) {                                   // relu on a plain A: it travels as one piece
            p.segA.n = 1;
            p.segA.begin[0] = 0;
            p.segA.begin[1] = (int)a->K;
            p.segA.ld[0] = a->lda;
            p.segA.base[0] = a->A;
        }
    }
    HAPMI_REQUIRE(!p.b_relu || (a->transA && !a->transB), HAPMI_EINVAL, "gemm: b_relu needs transA = 1, transB = 0");
    const hapmi_gemm_segments *bseg = a->B_segments;
    if (a->B_segments_list) {
        HAPMI_REQUIRE(lists && !a->B_segments, HAPMI_EINVAL, "gemm: B_segments_list goes with pointer lists (and without B_segments)");
        bseg = a->B_segments_list[0];
        HAPMI_REQUIRE(bseg, HAPMI_EINVAL, "gemm: null entry in B_segments_list");
    }
    rc_seg = fill_segments(p.segB, bseg, a->N, 64, 8, true, "B_segments");
    if (rc_seg) return rc_seg;
    if (p.segB.n > 0) {
        HAPMI_REQUIRE(!a->transB && (lists ? a->B_segments_list != nullptr : true), HAPMI_EINVAL,
                      "gemm: B_segments need transB = 0 (B stored [K, N])");
        for (int i = 1; i < p.segB.n; ++i) need.n_align = gcd64(need.n_align, p.segB.begin[i]);
        if (a->B_segments_list)
            for (int z = 0; z < p.n_list; ++z) {
                const hapmi_gemm_segments *sz = a->B_segments_list[z];
                HAPMI_REQUIRE(sz && sz->n == p.segB.n, HAPMI_EINVAL, "gemm: B_segments_list[%d] differs from the first entry", z);
                for (int i = 0; i < p.segB.n; ++i) {
                    HAPMI_REQUIRE(sz->begin[i] == bseg->begin[i] && sz->ld[i] == bseg->ld[i] && sz->base[i] &&
                                      ((uintptr_t)sz->base[i] % 16) == 0, HAPMI_EINVAL,
                                  "gemm: B_segments_list[%d] differs from the first entry or holds a bad base", z);
                    p.listSegB[z][i] = sz->base[i];
                }
            }
    }
    rc_seg = fill_segments(p.segC, a->C_segments, a->N, 64, 4, true, "C_segments");
    if (rc_seg) return rc_seg;
    rc_seg = fill_segments(p.segM, a->c_mask_segments, a->N, 64, 4, true, "c_mask_segments");
    if (rc_seg) return rc_seg;
    if (p.segC.n > 0) {
        HAPMI_REQUIRE(batch == 1 && !a->accumulate && !a->c_addend && !a->c_relu_mask, HAPMI_EINVAL,
                      "gemm: C_segments take one problem without accumulate / c_addend / c_relu_mask");
        for (int i = 1; i < p.segC.n; ++i) need.n_align = gcd64(need.n_align, p.segC.begin[i]);
    }
    if (p.segM.n > 0) {
        HAPMI_REQUIRE(p.segC.n == p.segM.n, HAPMI_EINVAL, "gemm: c_mask_segments go with C_segments of the same layout");
        for (int i = 0; i < p.segM.n; ++i)
            HAPMI_REQUIRE(p.segM.begin[i] == p.segC.begin[i] && p.segM.ld[i] == p.segC.ld[i], HAPMI_EINVAL,
                          "gemm: c_mask_segments go with C_segments of the same layout");
    }

    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
    bool prof = false;
    {
        std::lock_guard<std::mutex> lk(g_prof.mu);
        prof = g_prof.on;
        if (prof) {
            e0 = prof_event();
            e1 = prof_event();
            e2 = prof_event();
            prof = e0 && e1 && e2;
        }
    }
    if (prof) (void)hipEventRecord(e0, st);
    int rc;
    if (a->in_dtype == HAPMI_BF16 && a->out_dtype == HAPMI_BF16) rc = launch_typed<bf16_t, bf16_t>(p, a->transA, a->transB, batch, st, true, a->workspace, a->workspace_bytes, need);
    else if (a->in_dtype == HAPMI_BF16) rc = launch_typed<bf16_t, float>(p, a->transA, a->transB, batch, st, true, a->workspace, a->workspace_bytes, need);
    else if (a->out_dtype == HAPMI_F32) rc = launch_typed<float, float>(p, a->transA, a->transB, batch, st, false, a->workspace, a->workspace_bytes, need);
    else rc = launch_typed<float, bf16_t>(p, a->transA, a->transB, batch, st, false, a->workspace, a->workspace_bytes, need);
    if (prof) {
        (void)hipEventRecord(e1, st);
        (void)hipEventRecord(e2, st);                 // an empty bracket right behind: what two event records cost by themselves
        std::lock_guard<std::mutex> lk(g_prof.mu);
        g_prof.pending.push_back(ProfState::Bracket{e0, e1, e2});
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

extern "C" int hapmi_gemm_plan_set(int64_t M, int64_t N, int64_t K, int64_t batch, int transA, int transB, int in_dtype,
                                   int out_dtype, int tile_config, int k_splits) {
    HAPMI_REQUIRE(hapmi_dtype_ok(in_dtype) && hapmi_dtype_ok(out_dtype), HAPMI_EINVAL, "gemm_plan_set: bad dtype");
    HAPMI_REQUIRE(tile_config < kNumCfg && k_splits >= 1 && k_splits <= 64, HAPMI_EINVAL,
                  "gemm_plan_set: configuration %d / splits %d out of range", tile_config, k_splits);
    const PlanKey key(M, N, K, batch, (int)(transA != 0), (int)(transB != 0), in_dtype, out_dtype);
    std::lock_guard<std::mutex> lk(g_plans_mu);
    if (tile_config < 0) g_plans.erase(key);
    else g_plans[key] = std::make_pair(tile_config, k_splits);
    return HAPMI_OK;
}

extern "C" int hapmi_gemm_plan_clear(void) {
    std::lock_guard<std::mutex> lk(g_plans_mu);
    g_plans.clear();
    return HAPMI_OK;
}

extern "C" int hapmi_prof_gemm_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof.mu);
    g_prof.on = on != 0;
    return HAPMI_OK;
}

extern "C" int hapmi_prof_gemm_collect(double *ms, int64_t *launches, double *flops, double *empty_ms) {
    std::lock_guard<std::mutex> lk(g_prof.mu);
    double total = 0.0, empty = 0.0;
    for (auto &br : g_prof.pending) {
        if (hipEventSynchronize(br.e2) != hipSuccess) return hapmi_set_error(HAPMI_ELAUNCH, "prof: event sync failed");
        float t = 0.f, t0 = 0.f;
        if (hipEventElapsedTime(&t, br.e0, br.e1) != hipSuccess || hipEventElapsedTime(&t0, br.e1, br.e2) != hipSuccess)
            return hapmi_set_error(HAPMI_ELAUNCH, "prof: elapsed time failed");
        total += t;
        empty += t0;
        g_prof.pool.push_back(br.e0);
        g_prof.pool.push_back(br.e1);
        g_prof.pool.push_back(br.e2);
    }
    g_prof.pending.clear();
    if (ms) *ms = total;
    if (empty_ms) *empty_ms = empty;
    if (launches) *launches = g_prof.launches;
    if (flops) *flops = g_prof.flops;
    g_prof.flops = 0.0;
    g_prof.launches = 0;
    return HAPMI_OK;
}
