// Top-2 and switch (top-1) gating in index form and the dispatch / combine row gathers of the MoE layer.
// Integer routing (expert index, slot, token_of_slot) is exact; gate values are float32.
#include "common.h"

namespace {

constexpr int GATE_THREADS = 256;
constexpr int GATE_MAX_E = 64;

// Gating runs as two launches.  gate_choice_kernel, one thread per token: softmax over the experts, the two largest
// probabilities (ties -> lower expert index) as index / gate records.  gate_position_kernel, one wave per (batch
// row, expert): walks the row's S tokens in order, 64 at a time, and gives every token that chose this expert its
// 1-based position among the row's earlier choices of the same expert (a ballot and a population count per 64
// tokens); first the first choices, then the second choices, offset by the SUM of the expert's first-choice positions
// (n(n+1)/2), as the reference adds sum(position_in_expert[:, :, 0, :]) rather than the count.  A position >= C drops
// the choice (slot 0).  B * E waves work in parallel where the positions of a row are a serial count.
// TOP_K = 1 is switch gating: first choices only; the second entry of every record is written as a dropped choice
// (gate 0, slot 0), so the dispatch / combine kernels and the gate backward serve both kinds of record.
template <int TOP_K>
__global__ __launch_bounds__(GATE_THREADS) void gate_choice_kernel(const float *logits, float *probs, int32_t *index,
                                                                 int32_t *slot, float *gate, int64_t n_tok, int E) {
    const int64_t tok = (int64_t)blockIdx.x * GATE_THREADS + threadIdx.x;
    if (tok >= n_tok) return;
    const float *lg = logits + tok * E;
    float m = -INFINITY;
    for (int e = 0; e < E; ++e) m = fmaxf(m, lg[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf(lg[e] - m);
    const float inv = 1.0f / sum;
    int i0 = 0, i1 = -1;
    float p0 = -1.f, p1 = -1.f;
    for (int e = 0; e < E; ++e) {
        const float pe = expf(lg[e] - m) * inv;
        probs[tok * E + e] = pe;
        if (pe > p0) {
            p1 = p0; i1 = i0;
            p0 = pe; i0 = e;
        } else if (pe > p1) {
            p1 = pe; i1 = e;
        }
    }
    if (i1 < 0) i1 = (i0 + 1) % E;      // only with NaN logits; gate stays -1, so the choice is dropped
    index[tok * 2 + 0] = i0;
    index[tok * 2 + 1] = i1;
    gate[tok * 2 + 0] = p0;
    gate[tok * 2 + 1] = TOP_K == 2 ? p1 : 0.f;
    if (TOP_K == 1) slot[tok * 2 + 1] = 0;
}

template <int TOP_K>
__global__ __launch_bounds__(GATE_THREADS) void gate_position_kernel(const int32_t *index, const float *gate, int32_t *slot,
                                                                   int32_t *token_of_slot, int B, int S, int E, int C) {
    const int lane = threadIdx.x & 63;
    const int64_t pair = (int64_t)blockIdx.x * (GATE_THREADS / 64) + (threadIdx.x >> 6);      // (b, e), wave-uniform
    if (pair >= (int64_t)B * E) return;
    const int b = (int)(pair / E), e = (int)(pair % E);
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int32_t *tos = token_of_slot + ((int64_t)b * E + e) * C;
    for (int c = lane; c < C; c += 64) tos[c] = -1;
    long long run = 0, offset = 0;
#pragma unroll
    for (int pass = 0; pass < TOP_K; ++pass) {
        for (int s0 = 0; s0 < S; s0 += 64) {
            const int s = s0 + lane;
            const int64_t rec = ((int64_t)b * S + s) * 2 + pass;
            const bool mine = s < S && index[rec] == e;
            const unsigned long long bal = __ballot(mine);
            if (mine) {
                const long long pos = run + __popcll(bal & lt_mask) + 1 + offset;
                const int sl = (pos < C && gate[rec] > 0.f) ? (int)pos : 0;
                slot[rec] = sl;
                if (sl > 0) tos[sl] = s;             // slots 1 .. C - 1 of this wave's own (b, e): behind its own fill
            }
            run += __popcll(bal);
        }
        offset = run * (run + 1) / 2;
        run = 0;
    }
}

__global__ __launch_bounds__(256) void top2_gate_bwd_kernel(const float *probs, const int32_t *index, const int32_t *slot,
                                                          const float *dgate, float *dlogits, int64_t n_tok, int E) {
    const int64_t tok = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (tok >= n_tok) return;
    const int i0 = index[tok * 2], i1 = index[tok * 2 + 1];
    const float g0 = slot[tok * 2] > 0 ? dgate[tok * 2] : 0.f;
    const float g1 = slot[tok * 2 + 1] > 0 ? dgate[tok * 2 + 1] : 0.f;
    const float *p = probs + tok * E;
    const float dot = p[i0] * g0 + p[i1] * g1;
    for (int e = 0; e < E; ++e) {
        const float dp = (e == i0 ? g0 : 0.f) + (e == i1 ? g1 : 0.f);
        dlogits[tok * E + e] = p[e] * (dp - dot);
    }
}

__global__ __launch_bounds__(256) void top2_densify_kernel(const int32_t *index, const int32_t *slot, const float *gate,
                                                         float *dispatch, float *combine, int64_t n_tok, int E, int C) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_tok * 2) return;
    const int sl = slot[i];
    if (sl <= 0) return;
    const int64_t tok = i >> 1;
    const int64_t at = (tok * E + index[i]) * C + sl;
    combine[at] = gate[i];
    dispatch[at] = 1.0f;
}

// ---- row gathers: one wave per row of d elements, 16-byte vectors ------------------------------
template <typename T> struct RowVec {
    static constexpr int EPV = Vec16<T>::N;
};

// The device's share of the dense [B, S, E, C] routing tensors is a window in each of the three dimensions that the
// einsums may be split along: experts [e_lo, e_lo + E_loc), capacity slots [c_lo, c_lo + C_loc) and positions
// [s_lo, s_lo + S_loc).  Expert-major activations hold [E_loc, B, C_loc, d], token tensors [B, S_loc, d]; the routing
// records always cover all S positions.
//
// expert_in[e_loc, b, c, :] = x[b, token_of_slot[b, e_lo + e_loc, c_lo + c] - s_lo, :], or 0 for an empty slot or a
// token outside the window of positions
template <typename T>
__global__ __launch_bounds__(256) void moe_dispatch_kernel(const T *x, const int32_t *token_of_slot, T *expert_in, int B,
                                                         int S, int E, int C, int d, int e_lo, int E_loc, int c_lo,
                                                         int C_loc, int s_lo, int S_loc) {
    constexpr int EPV = Vec16<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)E_loc * B * C_loc) return;
    const int c = (int)(row % C_loc);
    const int b = (int)((row / C_loc) % B);
    const int el = (int)(row / ((int64_t)C_loc * B));
    const int tok = token_of_slot[((int64_t)b * E + e_lo + el) * C + c_lo + c];
    Vec16<T> *dst = (Vec16<T> *)(expert_in + row * d);
    if (tok >= s_lo && tok < s_lo + S_loc) {
        const Vec16<T> *src = (const Vec16<T> *)(x + ((int64_t)b * S_loc + tok - s_lo) * d);
        for (int i = lane; i < d / EPV; i += 64) dst[i] = src[i];
    } else {
        Vec16<T> z;
#pragma unroll
        for (int k = 0; k < EPV; ++k) z.set(k, 0.f);
        for (int i = lane; i < d / EPV; i += 64) dst[i] = z;
    }
}

// out[b, s - s_lo, :] (+)= sum_k w_k * src[e_k - e_lo, b, slot_k - c_lo, :] over kept local choices; w_k = gate_k or 1
template <typename T, bool WEIGHTED>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T *src, const int32_t *index, const int32_t *slot,
                                                        const float *gate, T *out, int B, int S, int C, int d, int e_lo,
                                                        int E_loc, int c_lo, int C_loc, int s_lo, int S_loc, int accumulate) {
    constexpr int EPV = Vec16<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t local = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);      // row of out: (b, s - s_lo)
    if (local >= (int64_t)B * S_loc) return;
    const int b = (int)(local / S_loc);
    const int64_t tok = (int64_t)b * S + s_lo + (local - (int64_t)b * S_loc); // the token's row in the routing records
    const Vec16<T> *rows[2] = {nullptr, nullptr};
    float w[2] = {0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int e = index[tok * 2 + k] - e_lo, sl = slot[tok * 2 + k];
        if (sl > 0 && sl < C && sl >= c_lo && sl < c_lo + C_loc && e >= 0 && e < E_loc) {
            rows[k] = (const Vec16<T> *)(src + (((int64_t)e * B + b) * C_loc + sl - c_lo) * d);
            w[k] = WEIGHTED ? gate[tok * 2 + k] : 1.0f;
        }
    }
    Vec16<T> *dst = (Vec16<T> *)(out + local * d);
    for (int i = lane; i < d / EPV; i += 64) {
        float acc[EPV];
#pragma unroll
        for (int k = 0; k < EPV; ++k) acc[k] = 0.f;
        if (accumulate) {
            const Vec16<T> o = dst[i];
#pragma unroll
            for (int k = 0; k < EPV; ++k) acc[k] = o.get(k);
        }
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if (rows[q]) {
                const Vec16<T> v = rows[q][i];
#pragma unroll
                for (int k = 0; k < EPV; ++k) acc[k] += w[q] * v.get(k);
            }
        }
        Vec16<T> r;
#pragma unroll
        for (int k = 0; k < EPV; ++k) r.set(k, acc[k]);
        dst[i] = r;
    }
}

// d_expert_out[e_loc, b, c, :] = gate * dout[b, token, :] (0 for empty slots)
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_bwd_rows_kernel(const T *dout, const int32_t *index, const float *gate,
                                                                 const int32_t *token_of_slot, T *d_expert_out, int B,
                                                                 int S, int E, int C, int d, int e_lo, int E_loc,
                                                                 int c_lo, int C_loc, int s_lo, int S_loc) {
    constexpr int EPV = Vec16<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)E_loc * B * C_loc) return;
    const int c = (int)(row % C_loc);
    const int b = (int)((row / C_loc) % B);
    const int el = (int)(row / ((int64_t)C_loc * B));
    const int tok = token_of_slot[((int64_t)b * E + e_lo + el) * C + c_lo + c];
    Vec16<T> *dst = (Vec16<T> *)(d_expert_out + row * d);
    float w = 0.f;
    const Vec16<T> *src = nullptr;
    if (tok >= s_lo && tok < s_lo + S_loc) {
        const int64_t t = (int64_t)b * S + tok;
        w = (index[t * 2] == e_lo + el) ? gate[t * 2] : gate[t * 2 + 1];
        src = (const Vec16<T> *)(dout + ((int64_t)b * S_loc + tok - s_lo) * d);
    }
    for (int i = lane; i < d / EPV; i += 64) {
        Vec16<T> r;
        if (src) {
            const Vec16<T> v = src[i];
#pragma unroll
            for (int k = 0; k < EPV; ++k) r.set(k, w * v.get(k));
        } else {
#pragma unroll
            for (int k = 0; k < EPV; ++k) r.set(k, 0.f);
        }
        dst[i] = r;
    }
}

// dgate[b, s, k] = <dout[b, s - s_lo, :], expert_out[e_k - e_lo, b, slot_k - c_lo, :]>, 0 for a token or a choice outside
// the windows (dgate covers all S positions)
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_bwd_gate_kernel(const T *dout, const T *expert_out, const int32_t *index,
                                                                 const int32_t *slot, float *dgate, int B, int S, int C,
                                                                 int d, int e_lo, int E_loc, int c_lo, int C_loc, int s_lo,
                                                                 int S_loc) {
    constexpr int EPV = Vec16<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t tok = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= (int64_t)B * S) return;
    const int b = (int)(tok / S);
    const int sp = (int)(tok - (int64_t)b * S) - s_lo;                         // position inside the window
    const bool mine = sp >= 0 && sp < S_loc;
    const Vec16<T> *g = (const Vec16<T> *)(dout + ((int64_t)b * S_loc + (mine ? sp : 0)) * d);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int e = index[tok * 2 + k] - e_lo, sl = slot[tok * 2 + k];
        float acc = 0.f;
        if (mine && sl > 0 && sl < C && sl >= c_lo && sl < c_lo + C_loc && e >= 0 && e < E_loc) {
            const Vec16<T> *r = (const Vec16<T> *)(expert_out + (((int64_t)e * B + b) * C_loc + sl - c_lo) * d);
            for (int i = lane; i < d / EPV; i += 64) {
                const Vec16<T> a = g[i], v = r[i];
#pragma unroll
                for (int q = 0; q < EPV; ++q) acc += a.get(q) * v.get(q);
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) dgate[tok * 2 + k] = acc;
    }
}

int check_moe(const char *name, int64_t B, int64_t S, int64_t E, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc,
              int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc, int dtype) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "%s: bad dtype", name);
    HAPMI_REQUIRE(B >= 0 && S >= 1 && E >= 2 && C >= 1 && d >= 1 && e_lo >= 0 && E_loc >= 0 && e_lo + E_loc <= E,
                  HAPMI_EINVAL, "%s: bad shape", name);
    HAPMI_REQUIRE(c_lo >= 0 && C_loc >= 0 && c_lo + C_loc <= C, HAPMI_EINVAL, "%s: capacity range [%lld, %lld) outside [0, %lld)",
                  name, (long long)c_lo, (long long)(c_lo + C_loc), (long long)C);
    HAPMI_REQUIRE(s_lo >= 0 && S_loc >= 0 && s_lo + S_loc <= S, HAPMI_EINVAL, "%s: range of positions [%lld, %lld) outside [0, %lld)",
                  name, (long long)s_lo, (long long)(s_lo + S_loc), (long long)S);
    const int64_t epv = dtype == HAPMI_F32 ? 4 : 8;
    HAPMI_REQUIRE(d % epv == 0, HAPMI_EALIGN, "%s: d must be a multiple of %lld", name, (long long)epv);
    HAPMI_REQUIRE(B * S < (1ll << 31) && E_loc * B * C_loc < (1ll << 31), HAPMI_ELIMIT, "%s: too many rows", name);
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_top2_gate(const float *logits, float *probs, int32_t *index, int32_t *slot, float *gate,
                               int32_t *token_of_slot, int64_t B, int64_t S, int64_t E, int64_t C,
                               hapmi_stream_t stream) {
    HAPMI_REQUIRE(B >= 0 && S >= 1 && C >= 1, HAPMI_EINVAL, "top2_gate: bad shape");
    HAPMI_REQUIRE(E >= 2 && E <= GATE_MAX_E, HAPMI_ELIMIT, "top2_gate: n_expert %lld outside 2..%d", (long long)E, GATE_MAX_E);
    HAPMI_REQUIRE(S < (1ll << 30) && B < (1ll << 31) && E * C < (1ll << 31), HAPMI_ELIMIT, "top2_gate: shape too large");
    if (B == 0) return HAPMI_OK;
    HAPMI_REQUIRE(logits && probs && index && slot && gate && token_of_slot, HAPMI_EINVAL, "top2_gate: null pointer");
    hipLaunchKernelGGL(gate_choice_kernel<2>, dim3((unsigned)hapmi_cdiv(B * S, GATE_THREADS)), dim3(GATE_THREADS), 0,
                       (hipStream_t)stream, logits, probs, index, slot, gate, B * S, (int)E);
    hipLaunchKernelGGL(gate_position_kernel<2>, dim3((unsigned)hapmi_cdiv(B * E, GATE_THREADS / 64)), dim3(GATE_THREADS), 0,
                       (hipStream_t)stream, index, gate, slot, token_of_slot, (int)B, (int)S, (int)E, (int)C);
    HAPMI_CHECK_LAUNCH("top2_gate");
    return HAPMI_OK;
}

extern "C" int hapmi_switch_gate(const float *logits, float *probs, int32_t *index, int32_t *slot, float *gate,
                                 int32_t *token_of_slot, int64_t B, int64_t S, int64_t E, int64_t C,
                                 hapmi_stream_t stream) {
    HAPMI_REQUIRE(B >= 0 && S >= 1 && C >= 1, HAPMI_EINVAL, "switch_gate: bad shape");
    HAPMI_REQUIRE(E >= 2 && E <= GATE_MAX_E, HAPMI_ELIMIT, "switch_gate: n_expert %lld outside 2..%d", (long long)E, GATE_MAX_E);
    HAPMI_REQUIRE(S < (1ll << 30) && B < (1ll << 31) && E * C < (1ll << 31), HAPMI_ELIMIT, "switch_gate: shape too large");
    if (B == 0) return HAPMI_OK;
    HAPMI_REQUIRE(logits && probs && index && slot && gate && token_of_slot, HAPMI_EINVAL, "switch_gate: null pointer");
    hipLaunchKernelGGL(gate_choice_kernel<1>, dim3((unsigned)hapmi_cdiv(B * S, GATE_THREADS)), dim3(GATE_THREADS), 0,
                       (hipStream_t)stream, logits, probs, index, slot, gate, B * S, (int)E);
    hipLaunchKernelGGL(gate_position_kernel<1>, dim3((unsigned)hapmi_cdiv(B * E, GATE_THREADS / 64)), dim3(GATE_THREADS), 0,
                       (hipStream_t)stream, index, gate, slot, token_of_slot, (int)B, (int)S, (int)E, (int)C);
    HAPMI_CHECK_LAUNCH("switch_gate");
    return HAPMI_OK;
}

extern "C" int hapmi_top2_gate_bwd(const float *probs, const int32_t *index, const int32_t *slot, const float *dgate,
                                   float *dlogits, int64_t B, int64_t S, int64_t E, hapmi_stream_t stream) {
    HAPMI_REQUIRE(B >= 0 && S >= 1 && E >= 2, HAPMI_EINVAL, "top2_gate_bwd: bad shape");
    if (B == 0) return HAPMI_OK;
    HAPMI_REQUIRE(probs && index && slot && dgate && dlogits, HAPMI_EINVAL, "top2_gate_bwd: null pointer");
    hipLaunchKernelGGL(top2_gate_bwd_kernel, dim3((unsigned)hapmi_cdiv(B * S, 256)), dim3(256), 0, (hipStream_t)stream,
                       probs, index, slot, dgate, dlogits, B * S, (int)E);
    HAPMI_CHECK_LAUNCH("top2_gate_bwd");
    return HAPMI_OK;
}

extern "C" int hapmi_top2_densify(const int32_t *index, const int32_t *slot, const float *gate, float *dispatch,
                                  float *combine, int64_t B, int64_t S, int64_t E, int64_t C, hapmi_stream_t stream) {
    HAPMI_REQUIRE(B >= 0 && S >= 1 && E >= 2 && C >= 1, HAPMI_EINVAL, "top2_densify: bad shape");
    if (B == 0) return HAPMI_OK;
    HAPMI_REQUIRE(index && slot && gate && dispatch && combine, HAPMI_EINVAL, "top2_densify: null pointer");
    int rc = hapmi_fill_zero(dispatch, B * S * E * C * 4, stream);
    if (rc) return rc;
    rc = hapmi_fill_zero(combine, B * S * E * C * 4, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(top2_densify_kernel, dim3((unsigned)hapmi_cdiv(B * S * 2, 256)), dim3(256), 0, (hipStream_t)stream,
                       index, slot, gate, dispatch, combine, B * S, (int)E, (int)C);
    HAPMI_CHECK_LAUNCH("top2_densify");
    return HAPMI_OK;
}

extern "C" int hapmi_moe_dispatch(const void *x, const int32_t *token_of_slot, void *expert_in, int64_t B, int64_t S,
                                  int64_t E, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc, int64_t c_lo,
                                  int64_t C_loc, int64_t s_lo, int64_t S_loc, int dtype, hapmi_stream_t stream) {
    int rc = check_moe("moe_dispatch", B, S, E, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, dtype);
    if (rc) return rc;
    const int64_t rows = E_loc * B * C_loc;
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE((x || S_loc == 0) && token_of_slot && expert_in, HAPMI_EINVAL, "moe_dispatch: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(rows, 4));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((moe_dispatch_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, (const float *)x, token_of_slot, (float *)expert_in, (int)B, (int)S, (int)E, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
    else
        hipLaunchKernelGGL((moe_dispatch_kernel<bf16_t>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t *)x, token_of_slot, (bf16_t *)expert_in, (int)B, (int)S, (int)E, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
    HAPMI_CHECK_LAUNCH("moe_dispatch");
    return HAPMI_OK;
}

extern "C" int hapmi_moe_combine(const void *expert_out, const int32_t *index, const int32_t *slot, const float *gate,
                                 void *out, int64_t B, int64_t S, int64_t C, int64_t d, int64_t e_lo, int64_t E_loc,
                                 int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc, int dtype, hapmi_stream_t stream) {
    int rc = check_moe("moe_combine", B, S, e_lo + E_loc > 2 ? e_lo + E_loc : 2, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, dtype);
    if (rc) return rc;
    if (B == 0) return HAPMI_OK;
    if (S_loc == 0) return HAPMI_OK;
    HAPMI_REQUIRE(expert_out && index && slot && gate && out, HAPMI_EINVAL, "moe_combine: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(B * S_loc, 4));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((moe_combine_kernel<float, true>), grid, dim3(256), 0, (hipStream_t)stream, (const float *)expert_out, index, slot, gate, (float *)out, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc, 0);
    else
        hipLaunchKernelGGL((moe_combine_kernel<bf16_t, true>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t *)expert_out, index, slot, gate, (bf16_t *)out, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc, 0);
    HAPMI_CHECK_LAUNCH("moe_combine");
    return HAPMI_OK;
}

extern "C" int hapmi_moe_dispatch_bwd(const void *d_expert_in, const int32_t *index, const int32_t *slot,
                                      const float *gate, void *dx, int64_t B, int64_t S, int64_t C, int64_t d,
                                      int64_t e_lo, int64_t E_loc, int64_t c_lo, int64_t C_loc, int64_t s_lo, int64_t S_loc,
                                      int accumulate, int dtype, hapmi_stream_t stream) {
    int rc = check_moe("moe_dispatch_bwd", B, S, e_lo + E_loc > 2 ? e_lo + E_loc : 2, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, dtype);
    if (rc) return rc;
    if (B == 0) return HAPMI_OK;
    if (S_loc == 0) return HAPMI_OK;
    HAPMI_REQUIRE(d_expert_in && index && slot && gate && dx, HAPMI_EINVAL, "moe_dispatch_bwd: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(B * S_loc, 4));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((moe_combine_kernel<float, false>), grid, dim3(256), 0, (hipStream_t)stream, (const float *)d_expert_in, index, slot, gate, (float *)dx, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc, accumulate);
    else
        hipLaunchKernelGGL((moe_combine_kernel<bf16_t, false>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t *)d_expert_in, index, slot, gate, (bf16_t *)dx, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc, accumulate);
    HAPMI_CHECK_LAUNCH("moe_dispatch_bwd");
    return HAPMI_OK;
}

extern "C" int hapmi_moe_combine_bwd(const void *dout, const void *expert_out, const int32_t *index,
                                     const int32_t *slot, const float *gate, const int32_t *token_of_slot,
                                     void *d_expert_out, float *dgate, int64_t B, int64_t S, int64_t E, int64_t C,
                                     int64_t d, int64_t e_lo, int64_t E_loc, int64_t c_lo, int64_t C_loc, int64_t s_lo,
                                     int64_t S_loc, int dtype, hapmi_stream_t stream) {
    int rc = check_moe("moe_combine_bwd", B, S, E, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, dtype);
    if (rc) return rc;
    if (B == 0) return HAPMI_OK;
    HAPMI_REQUIRE((dout || S_loc == 0) && expert_out && index && slot && gate && token_of_slot && d_expert_out && dgate, HAPMI_EINVAL,
                  "moe_combine_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int64_t rows = E_loc * B * C_loc;
    dim3 grid_rows((unsigned)hapmi_cdiv(rows > 0 ? rows : 1, 4)), grid_tok((unsigned)hapmi_cdiv(B * S, 4));
    if (dtype == HAPMI_F32) {
        if (rows) hipLaunchKernelGGL((moe_combine_bwd_rows_kernel<float>), grid_rows, dim3(256), 0, st, (const float *)dout, index, gate, token_of_slot, (float *)d_expert_out, (int)B, (int)S, (int)E, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
        hipLaunchKernelGGL((moe_combine_bwd_gate_kernel<float>), grid_tok, dim3(256), 0, st, (const float *)dout, (const float *)expert_out, index, slot, dgate, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
    } else {
        if (rows) hipLaunchKernelGGL((moe_combine_bwd_rows_kernel<bf16_t>), grid_rows, dim3(256), 0, st, (const bf16_t *)dout, index, gate, token_of_slot, (bf16_t *)d_expert_out, (int)B, (int)S, (int)E, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
        hipLaunchKernelGGL((moe_combine_bwd_gate_kernel<bf16_t>), grid_tok, dim3(256), 0, st, (const bf16_t *)dout, (const bf16_t *)expert_out, index, slot, dgate, (int)B, (int)S, (int)C, (int)d, (int)e_lo, (int)E_loc, (int)c_lo, (int)C_loc, (int)s_lo, (int)S_loc);
    }
    HAPMI_CHECK_LAUNCH("moe_combine_bwd");
    return HAPMI_OK;
}
