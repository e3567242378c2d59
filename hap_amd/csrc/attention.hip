// Fused scaled-dot-product attention for bf16, head_dim 64, on the packed projection qkv[b, S, 3*H*64].
//
// Everything is computed "transposed" so that the softmax dimension lives inside a lane:
//   forward / dQ : S^T[kv][q] = K Q^T   -> each lane owns one query column (lane % 32) and 32 kv rows per tile,
//                  so row max / row sum are per-lane loops plus one exchange with lane ^ 32;
//   dK / dV      : S[q][kv]   = Q K^T   -> each lane owns one kv column.
// The probability tile leaves the MFMA in accumulator layout (lane = column, registers = rows); it is fed to
// the next MFMA as its B operand straight from registers by choosing the k-order (slot (h, j) of step s is row
// 16 s + 8 (j / 4) + 4 h + j % 4), and the matching A operand is read from LDS in that same order.
// K / V / Q / dO tiles sit in LDS row-major, [row][128 B of d], 16-byte chunks XOR-swizzled with aswz(row).
// Fragments along d (k = d) are plain 16-byte reads; fragments of the TRANSPOSED tile (k = tile rows: V^T for
// P V, K^T for dQ, Q^T and dO^T for dK / dV) are assembled from the same tile by transposing LDS reads
// (ds_read_b64_tr_b16), so no transposed copy is ever written.  aswz keeps both kinds of read and the
// row-wise tile stores free of bank conflicts: 16 lanes reading one chunk of 16 consecutive rows land in 16
// different 16-byte slots (row & 3 picks the 64-byte quarter, row >> 2 the slot), and the four 64-byte pieces
// of rows 4a .. 4a + 3 that a half wave touches in a transposing read fall into different quarters.
#include "common.h"
#include "dropout.h"
#include "tile.h"

namespace {

constexpr float LOG2E = 1.4426950408889634f;


constexpr int HD = 64;                 // head dimension (bf16: one 128-byte LDS row)
constexpr int TILE = 64;               // rows of the streamed operand per iteration
constexpr int AT_THREADS = 256;        // 4 waves, 32 rows of the stationary operand each
constexpr int TILE_BYTES = TILE * ROW_BYTES;

typedef Vec16<bf16_t> frag_t;

__device__ __forceinline__ int aswz(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

// standard operand fragment of k-step s: k = 16 s + 8 h .. + 8 of `row`
__device__ __forceinline__ frag_t frag_rowk(const char *tile, int row, int s, int h) {
    return *(const frag_t *)(tile + row * ROW_BYTES + ((((s << 1) | h) ^ aswz(row)) << 4));
}

// Fragment of the transposed tile in accumulator order: MFMA row = tile column col0 + lane % 32, slots j < 4 ->
// k = tile row 16 s + 4 h + j, slots j >= 4 -> tile row 16 s + 8 + 4 h + (j - 4).  Within a group of 16 lanes
// ds_read_b64_tr_b16 hands lane j the elements D[4 e + j / 4][j % 4], e = 0..3, of the 16 x 4 matrix whose row
// i is the 8 bytes at lane i's address: lane i points at tile row (first row + i / 4), columns 4 (i % 4) ...
struct TransposedReader {
    int base, cx;              // lane constants: byte offset of (row 4 h + i / 4, within-chunk part), swizzled chunk
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s lds_v4s;
    __device__ __forceinline__ TransposedReader() {
        const int lane = threadIdx.x & 63, i = lane & 15, half = (lane >> 4) & 1, h = lane >> 5, q = i >> 2;
        const int col = 16 * half + 4 * (i & 3);                  // + col0 (0 or 32: chunk + 0 or 4)
        base = (4 * h + q) * ROW_BYTES + (col & 7) * 2;
        cx = (col >> 3) ^ ((((q >> 1) & 1) << 2) | h);            // aswz(16 s + 4 h + q) = ((q >> 1) & 1) << 2 | h
    }
    __device__ __forceinline__ frag_t frag(const char *tile, int col0, int s) const {
        union { v4s h[2]; bf16x8 v; } u;
        // second read: rows + 8, whose swizzle differs by 2 (aswz low bits = (row >> 2) & 3)
        u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(tile + base + 16 * s * ROW_BYTES + ((cx ^ (col0 >> 3)) << 4)));
        u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)(tile + base + (16 * s + 8) * ROW_BYTES + ((cx ^ (col0 >> 3) ^ 2) << 4)));
        frag_t f;
        f.v = u.v;
        return f;
    }
};
// 8 rows (one k-step) of an accumulator tile as a B operand
__device__ __forceinline__ frag_t acc_to_b(const f32x16 &a, int sp) {
    frag_t f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f.v[j] = (bf16_t)a[sp * 8 + j];
    return f;
}
__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.f;
    return z;
}
__device__ __forceinline__ f32x16 mma(const frag_t &a, const frag_t &b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}
// row index inside a 32-row accumulator tile held in register r by a lane of half h
__device__ __forceinline__ int acc_row(int r, int h) { return ((r >> 2) << 3) + (h << 2) + (r & 3); }

__device__ __forceinline__ frag_t load_row_frag(const bf16_t *row_ptr, bool valid, int s, int h) {
    frag_t f;
    if (valid) f = *(const frag_t *)(row_ptr + 16 * s + 8 * h);
    else {
#pragma unroll
        for (int j = 0; j < 8; ++j) f.v[j] = (bf16_t)0.f;
    }
    return f;
}

// One [64 rows][64 d] operand tile (memory [row][d], row stride ld) held as two 16-byte vectors per thread
// (rows 2 * (t / 8) and + 1, d chunk t % 8) on its way into the row-major LDS tile.  The thread's element offsets
// inside a tile and its LDS byte offsets are fixed for the kernel's lifetime; `base` (the tile's first element) is
// the same for every thread, so a load is one instruction on a scalar base and a constant vector offset, and
// full tiles skip the row checks.
struct PairLoader {
    frag_t v[2];
    int goff[2], soff[2];
    __device__ __forceinline__ PairLoader(int ld) {
        const int c8 = threadIdx.x & 7, r0 = (threadIdx.x >> 3) * 2;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            goff[i] = (r0 + i) * ld + c8 * 8;
            soff[i] = (r0 + i) * ROW_BYTES + ((c8 ^ aswz(r0 + i)) << 4);
        }
    }
    __device__ __forceinline__ void load(const bf16_t *base, int rows_left) {
        if (rows_left >= TILE) {
#pragma unroll
            for (int i = 0; i < 2; ++i) v[i] = *(const frag_t *)(base + goff[i]);
        } else {
            const int r0 = (threadIdx.x >> 3) * 2;
#pragma unroll
            for (int i = 0; i < 2; ++i) v[i] = load_row_frag(base + goff[i], r0 + i < rows_left, 0, 0);
        }
    }
    __device__ __forceinline__ void store_rows(char *lds) const {
#pragma unroll
        for (int i = 0; i < 2; ++i) *(frag_t *)(lds + soff[i]) = v[i];
    }
};

// One [64 rows][64 d] operand tile global -> LDS without a stop in registers (global_load_lds_dwordx4: every wave
// instruction fills 1024 contiguous LDS bytes = 8 tile rows, lane l landing in row l / 8, 16-byte slot l % 8).  The
// tile's swizzle is applied on the global side: the lane fetches the chunk that belongs in its slot.  Rows beyond the
// operand's end repeat its last row (finite values; the callers give such keys a probability of zero), since a
// transfer cannot be zero-filled.  The transfers are asynchronous: the caller counts them with s_waitcnt vmcnt (a
// wave's loads complete in issue order) and publishes the tile with a barrier.
struct DirectTileLoader {
    static constexpr int LOADS = 2;                            // wave instructions per tile (64 rows / 4 waves / 8 rows)
    int row[LOADS], chunk[LOADS], ld;
    __device__ __forceinline__ DirectTileLoader(int ld_) : ld(ld_) {
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            row[i] = (i * 4 + wave) * 8 + (lane >> 3);
            chunk[i] = ((lane & 7) ^ aswz(row[i])) * 8;
        }
    }
    __device__ __forceinline__ void issue(const bf16_t *base, int rows_left, char *lds_tile) const {
        typedef __attribute__((address_space(3))) char lds_char;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int r = row[i] < rows_left ? row[i] : rows_left - 1;
            const bf16_t *src = base + r * ld + chunk[i];
            const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_char *)(lds_tile + (i * 4 + wave) * 1024);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :
                         : "s"(lds_addr), "v"(src)
                         : "memory");
        }
    }
};

// One 4-byte word per thread global -> LDS (global_load_lds_dword: a wave instruction fills 256 contiguous LDS bytes,
// lane l landing in word l), into the thread's own slot lds_words[threadIdx.x]; asynchronous like the tile transfers.
__device__ __forceinline__ void issue_word(const uint32_t *src, uint32_t *lds_words) {
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_u32 *)(lds_words + wave * 64);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(lds_addr), "v"(src) : "memory");
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
// Which 128-row block and which (batch, head) a thread block works on.  Without a mask every block does the same
// work and the grid is taken as it is.  With the causal mask the work grows with the query block (falls with
// the key block): the blocks are renumbered so that the hardware, which starts blocks in the order of their
// linear index, starts the longest ones first and the short ones fill the tail.
template <bool CAUSAL> struct BlockOrder {
    __device__ __forceinline__ static int linear() { return (int)(blockIdx.y * gridDim.x + blockIdx.x); }
    // Without a mask: blocks are dealt round-robin over the 8 XCDs (each with an L2 of its own) in the order of
    // their linear index.  The row blocks of one (batch, head) stream the same K / V (Q / dO) tiles, so they are
    // given to the same XCD, next to each other in time: work item w = (XCD) * (items per XCD) + (turn on that XCD),
    // row block = w % row blocks.  The tiles then come from that XCD's L2 for all but the first of the blocks.
    __device__ __forceinline__ static int work_item() {
        const int n = (int)(gridDim.x * gridDim.y), l = linear();
        return (n % 8 == 0) ? (l % 8) * (n / 8) + l / 8 : l;
    }
    __device__ __forceinline__ static int row_block(bool work_grows_with_index) {
        if (!CAUSAL) return work_item() % (int)gridDim.x;
        const int i = linear() / (int)gridDim.y;
        return work_grows_with_index ? (int)gridDim.x - 1 - i : i;
    }
    __device__ __forceinline__ static int batch_head() { return CAUSAL ? linear() % (int)gridDim.y : work_item() / (int)gridDim.x; }
};

// CAUSAL: key j is visible to query i iff j <= i (the additive mask torch.triu(full(-inf), 1), models.py:72, 97),
// applied arithmetically; kv tiles that lie completely above the diagonal of the block's 128 queries are skipped.
// DROP: dropout of the probabilities (F.multi_head_attention_forward with dropout_p > 0, hap.rs:1257, 1307).  The
// keep decisions come as bit words (attn_keep_bits below): the row sums stay those of the undropped probabilities,
// the probabilities that multiply V are zeroed where the bit is clear, and the factor 1 / (1 - p) is applied to the
// output once at the end.
template <bool CAUSAL, bool DROP = false>
__global__ __launch_bounds__(AT_THREADS, 3) void attn_fwd_kernel(const bf16_t *qkv, const float *mask, bf16_t *out,
                                                            float *lse, int S, int H, float scale,
                                                            const uint32_t *keep_rows = nullptr, float keep_scale = 1.f) {
    // three K and three V tiles: one is multiplied while the next two are on their way global -> LDS
    constexpr int NST = 3;
    __shared__ __attribute__((aligned(16))) char Ks3[NST][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char Vs3[NST][TILE_BYTES];
    // DROP: each thread's keep word of a tile travels with the tile (one 4-byte transfer per thread, landing in the
    // thread's own slot), so it is counted by the same wait and needs no wait of its own
    __shared__ __attribute__((aligned(16))) uint32_t keep_s[DROP ? NST : 1][AT_THREADS];
    const TransposedReader tr;
    const int E = H * HD, ld = 3 * E;
    const int blk = BlockOrder<CAUSAL>::row_block(true), bh = BlockOrder<CAUSAL>::batch_head();
    const int b = bh / H, hh = bh % H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 31, h = lane >> 5;
    const int q = blk * 128 + wave * 32 + c;
    const bool qok = q < S;
    const bf16_t *Q = qkv + (int64_t)b * S * ld + hh * HD;
    const bf16_t *K = Q + E, *V = Q + 2 * E;

    frag_t qf[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) qf[s] = load_row_frag(Q + (int64_t)q * ld, qok, s, h);

    f32x16 ot[2] = {zero16(), zero16()};
    float m = -INFINITY, lsum = 0.f;
    const DirectTileLoader ldr(ld);
    const bool vec_mask = mask && ((S & 3) == 0);
    // Softmax is VALU work next to the MFMAs (32 scores per lane and kv tile), so the common tile (no additive
    // mask, every query and key of the tile valid and, if causal, visible) takes a short path: maximum over the raw
    // scores, then one fused multiply-add and one exp2 per score.
    const float sl2 = scale * LOG2E;
    const bool plain_block = !mask && blk * 128 + 128 <= S;

    // K / V tiles go global -> LDS directly, two tiles ahead of the one that is multiplied: a tile's transfers have
    // two iterations to arrive (the tiles come from the memory-side cache or HBM the first time an XCD touches them,
    // which takes longer than one iteration).  A wave's transfers complete in issue order, so tile i has landed once
    // at most the 2 x LOADS transfers of tile i + 1 are outstanding; the barrier then publishes every wave's part and
    // tells that everyone is done with tile i - 1, whose buffers take tile i + 2.
    const int q_blk_end = blk * 128 + 128;
    const int kv_end = (CAUSAL && q_blk_end < S) ? q_blk_end : S;
    constexpr int PER_TILE = 2 * DirectTileLoader::LOADS + (DROP ? 1 : 0);
    static_assert(2 * DirectTileLoader::LOADS == 4, "the waits below are written for four (five) transfers per tile");
    const int n_kt = (S + TILE - 1) / TILE;
    const uint32_t *keep_row = DROP ? keep_rows + ((int64_t)bh * S + (qok ? q : S - 1)) * n_kt * 2 + h : nullptr;
    auto issue_tile = [&](int kv0, int bufi) {
        ldr.issue(K + (int64_t)kv0 * ld, S - kv0, Ks3[bufi]);
        ldr.issue(V + (int64_t)kv0 * ld, S - kv0, Vs3[bufi]);
        if constexpr (DROP) issue_word(keep_row + (kv0 / TILE) * 2, &keep_s[bufi][0]);
    };
    issue_tile(0, 0);
    if (TILE < kv_end) issue_tile(TILE, 1);
    // The query fragments are consumed here, before the loop: otherwise the wait for their loads would sit at their
    // first use inside the loop body, as a wait for ALL outstanding loads in every iteration (the compiler does not
    // count the transfers above), and no tile would ever be in flight across an iteration.
#pragma unroll
    for (int s = 0; s < 4; ++s) asm volatile("" : "+v"(qf[s].v));
    int buf = 0;
    for (int kv0 = 0; kv0 < kv_end; kv0 += TILE) {
        if (kv0 + TILE < kv_end) __builtin_amdgcn_s_waitcnt(0x0F70 | PER_TILE);   // vmcnt(4 / 5): only tile i + 1 may be outstanding
        else __builtin_amdgcn_s_waitcnt(0x0F70);                       // vmcnt(0)
        __syncthreads();
        if (kv0 + 2 * TILE < kv_end) issue_tile(kv0 + 2 * TILE, buf == 0 ? 2 : buf - 1);
        const char *Ks = Ks3[buf], *Vs = Vs3[buf];
        uint32_t keep = 0xffffffffu;                               // this lane's 32 keys of the tile, bit = register index
        if constexpr (DROP) keep = keep_s[buf][threadIdx.x];
        // all fragment reads of the tile are issued before the first MFMA waits for one
        frag_t kf[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 4; ++s) kf[t][s] = frag_rowk(Ks, t * 32 + c, s, h);
        f32x16 st[2] = {zero16(), zero16()};
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int t = 0; t < 2; ++t) st[t] = mma(kf[t][s], qf[s], st[t]);

        float alpha, psum = 0.f;
        if (plain_block && kv0 + TILE <= S && (!CAUSAL || kv0 + TILE - 1 <= blk * 128)) {
            float mx = st[0][0];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[t][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m, mx * scale);            // finite: every score of the tile is
            const float nm = -m_new * LOG2E;
            alpha = __builtin_amdgcn_exp2f(fmaf(m, LOG2E, nm));   // m = -inf before the first tile: 0
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(st[t][r], sl2, nm));
                    st[t][r] = p;
                    psum += p;
                }
            m = m_new;
        } else {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int kv = kv0 + t * 32 + g * 8 + h * 4;
                    float mk[4] = {0.f, 0.f, 0.f, 0.f};
                    if (mask && qok) {
                        if (vec_mask && kv + 4 <= S) {
                            const f32x4 mv = *(const f32x4 *)(mask + (int64_t)q * S + kv);
#pragma unroll
                            for (int e = 0; e < 4; ++e) mk[e] = mv[e];
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (kv + e < S) mk[e] = mask[(int64_t)q * S + kv + e];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = st[t][g * 4 + e] * scale + mk[e];
                        if (kv + e >= S || (CAUSAL && kv + e > q)) v = -INFINITY;
                        st[t][g * 4 + e] = v;
                        mx = fmaxf(mx, v);
                    }
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m, mx);
            const float msub = (m_new == -INFINITY) ? 0.f : m_new;
            alpha = (m_new == -INFINITY) ? 1.f : __expf(m - m_new);
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = __expf(st[t][r] - msub);
                    st[t][r] = p;
                    psum += p;
                }
            m = m_new;
        }
        lsum = lsum * alpha + psum;
        if constexpr (DROP) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) st[t][r] = (keep & (1u << (t * 16 + r))) ? st[t][r] : 0.f;
        }
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {          // the running maximum moved for some query
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 16; ++r) ot[u][r] *= alpha;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const frag_t pb = acc_to_b(st[s >> 1], s & 1);
#pragma unroll
            for (int u = 0; u < 2; ++u) ot[u] = mma(tr.frag(Vs, u * 32, s), pb, ot[u]);
        }
        buf = buf == NST - 1 ? 0 : buf + 1;
    }
    const float l = lsum + __shfl_xor(lsum, 32, 64);
    const float inv = (l > 0.f ? 1.0f / l : 0.f) * (DROP ? keep_scale : 1.f);
    if (qok) {
        bf16_t *orow = out + ((int64_t)b * S + q) * E + hh * HD;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16_t)(ot[u][g * 4 + e] * inv);
                *(bf16x4 *)(orow + u * 32 + g * 8 + h * 4) = o;
            }
        if (h == 0) lse[((int64_t)b * H + hh) * S + q] = m + __logf(l);
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: lanes own query columns, kv tiles are streamed
// ---------------------------------------------------------------------------------------------
template <bool CAUSAL, bool DROP = false>
__global__ __launch_bounds__(AT_THREADS, 2) void attn_bwd_dq_kernel(const bf16_t *qkv, const bf16_t *out, const bf16_t *dout,
                                                               const float *lse, float *delta, const float *mask,
                                                               bf16_t *dqkv, int S, int H, float scale,
                                                               const uint32_t *keep_rows = nullptr, float keep_scale = 1.f) {
    __shared__ __attribute__((aligned(16))) char Ks[TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char Vs[TILE_BYTES];
    const TransposedReader tr;
    const int E = H * HD, ld = 3 * E;
    const int blk = BlockOrder<CAUSAL>::row_block(true), bh = BlockOrder<CAUSAL>::batch_head();
    const int b = bh / H, hh = bh % H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 31, h = lane >> 5;
    const int q = blk * 128 + wave * 32 + c;
    const bool qok = q < S;
    const bf16_t *Q = qkv + (int64_t)b * S * ld + hh * HD;
    const bf16_t *K = Q + E, *V = Q + 2 * E;
    const bf16_t *dO = dout + (int64_t)b * S * E + hh * HD;

    frag_t qf[4], dof[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        qf[s] = load_row_frag(Q + (int64_t)q * ld, qok, s, h);
        dof[s] = load_row_frag(dO + (int64_t)q * E, qok, s, h);
    }
    const float lse_q = qok ? lse[((int64_t)b * H + hh) * S + q] : 0.f;
    // delta[b, h, q] = sum_d dO[q, d] * O[q, d]: each lane holds half of its query's dO row; the dK / dV kernel,
    // launched after this one, reads the values written here
    float delta_q = 0.f;
    {
        const bf16_t *O = out + (int64_t)b * S * E + hh * HD;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const frag_t of = load_row_frag(O + (int64_t)q * E, qok, s, h);
#pragma unroll
            for (int e = 0; e < 8; ++e) delta_q += (float)of.v[e] * (float)dof[s].v[e];
        }
        delta_q += __shfl_xor(delta_q, 32, 64);
        if (qok && h == 0) delta[((int64_t)b * H + hh) * S + q] = delta_q;
    }
    f32x16 dqt[2] = {zero16(), zero16()};
    PairLoader lk(ld), lv(ld);
    const bool vec_mask = mask && ((S & 3) == 0);
    // dS is kept without its factor `scale`, which the result gets once at the end; plain tiles (see the forward
    // kernel) take p = exp2(s * scale * log2 e - lse * log2 e) in two operations
    const float sl2 = scale * LOG2E, nl = -lse_q * LOG2E;
    const bool plain_block = !mask && blk * 128 + 128 <= S;

    const int q_blk_end = blk * 128 + 128;
    const int kv_end = (CAUSAL && q_blk_end < S) ? q_blk_end : S;
    lk.load(K, S);
    lv.load(V, S);
    // DROP: the lane's keep word of a tile (bit = register index) is fetched together with the tile
    const uint32_t *keep_row = DROP ? keep_rows + ((int64_t)bh * S + (qok ? q : S - 1)) * ((S + TILE - 1) / TILE) * 2 + h : nullptr;
    uint32_t keep = 0xffffffffu, keep_next = 0xffffffffu;
    if constexpr (DROP) keep_next = keep_row[0];
    for (int kv0 = 0; kv0 < kv_end; kv0 += TILE) {
        __syncthreads();
        lk.store_rows(Ks);
        lv.store_rows(Vs);
        if constexpr (DROP) keep = keep_next;
        __syncthreads();
        if (kv0 + TILE < kv_end) {
            const int nx = kv0 + TILE;
            lk.load(K + (int64_t)nx * ld, S - nx);
            lv.load(V + (int64_t)nx * ld, S - nx);
            if constexpr (DROP) keep_next = keep_row[(nx / TILE) * 2];
        }
        if (blk * 128 + wave * 32 >= S) continue;                  // a wave without queries only moves tiles and meets barriers

        // one 32-row kv block at a time keeps only one score / dP accumulator pair live
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (t == 1 && kv0 + 32 >= S) break;                    // the sequence ends in the tile's first half: no key here
            f32x16 st = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                st = mma(frag_rowk(Ks, t * 32 + c, s, h), qf[s], st);
                dp = mma(frag_rowk(Vs, t * 32 + c, s, h), dof[s], dp);
            }
            if constexpr (DROP) {                                  // d(P) = d(dropout(P)) * keep / (1 - p)
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = (keep & (1u << (t * 16 + r))) ? dp[r] * keep_scale : 0.f;
            }
            if (plain_block && kv0 + TILE <= S && (!CAUSAL || kv0 + TILE - 1 <= blk * 128)) {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    dp[r] = __builtin_amdgcn_exp2f(fmaf(st[r], sl2, nl)) * (dp[r] - delta_q);
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int kv = kv0 + t * 32 + g * 8 + h * 4;
                    float mk[4] = {0.f, 0.f, 0.f, 0.f};
                    if (mask && qok) {
                        if (vec_mask && kv + 4 <= S) {
                            const f32x4 mv = *(const f32x4 *)(mask + (int64_t)q * S + kv);
#pragma unroll
                            for (int e = 0; e < 4; ++e) mk[e] = mv[e];
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (kv + e < S) mk[e] = mask[(int64_t)q * S + kv + e];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = g * 4 + e;
                        float p = (qok && kv + e < S && !(CAUSAL && kv + e > q)) ? __expf(st[r] * scale + mk[e] - lse_q) : 0.f;
                        dp[r] = p * (dp[r] - delta_q);
                    }
                }
            }
#pragma unroll
            for (int sp = 0; sp < 2; ++sp) {
                const frag_t db = acc_to_b(dp, sp);
#pragma unroll
                for (int u = 0; u < 2; ++u) dqt[u] = mma(tr.frag(Ks, u * 32, t * 2 + sp), db, dqt[u]);
            }
        }
    }
    if (qok) {
        bf16_t *drow = dqkv + ((int64_t)b * S + q) * ld + hh * HD;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16_t)(dqt[u][g * 4 + e] * scale);
                *(bf16x4 *)(drow + u * 32 + g * 8 + h * 4) = o;
            }
    }
}

// ---------------------------------------------------------------------------------------------
// dK, dV: lanes own kv columns, query tiles are streamed
// ---------------------------------------------------------------------------------------------
template <bool CAUSAL, bool DROP = false>
__global__ __launch_bounds__(AT_THREADS, 2) void attn_bwd_dkv_kernel(const bf16_t *qkv, const bf16_t *dout, const float *lse,
                                                                const float *delta, const float *mask, bf16_t *dqkv,
                                                                int S, int H, float scale,
                                                                const uint32_t *keep_cols = nullptr, float keep_scale = 1.f) {
    __shared__ __attribute__((aligned(16))) char Qs[TILE_BYTES];
    __shared__ __attribute__((aligned(16))) char dOs[TILE_BYTES];
    const TransposedReader tr;
    __shared__ __attribute__((aligned(16))) float lse_s[TILE], delta_s[TILE];
    const int E = H * HD, ld = 3 * E;
    const int blk = BlockOrder<CAUSAL>::row_block(false), bh = BlockOrder<CAUSAL>::batch_head();
    const int b = bh / H, hh = bh % H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, c = lane & 31, h = lane >> 5;
    const int kv = blk * 128 + wave * 32 + c;
    const bool kok = kv < S;
    const bf16_t *Q = qkv + (int64_t)b * S * ld + hh * HD;
    const bf16_t *K = Q + E, *V = Q + 2 * E;
    const bf16_t *dO = dout + (int64_t)b * S * E + hh * HD;
    const float *lse_b = lse + ((int64_t)b * H + hh) * S, *delta_b = delta + ((int64_t)b * H + hh) * S;

    frag_t kf[4], vf[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        kf[s] = load_row_frag(K + (int64_t)kv * ld, kok, s, h);
        vf[s] = load_row_frag(V + (int64_t)kv * ld, kok, s, h);
    }
    f32x16 dvt[2] = {zero16(), zero16()}, dkt[2] = {zero16(), zero16()};
    PairLoader lq(ld), ldo(E);
    // log-sum-exps are staged times log2 e and dS is kept without its factor `scale` (applied once at the end)
    const float sl2 = scale * LOG2E;

    // causal: queries before the block's first key see none of its keys
    const int q_begin = CAUSAL ? blk * 128 : 0;
    lq.load(Q + (int64_t)q_begin * ld, S - q_begin);
    ldo.load(dO + (int64_t)q_begin * E, S - q_begin);
    // DROP: the lane's two keep words of a query tile (one per 32 queries, bit = query) are fetched with the tile
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 *keep_col = DROP ? (const u32x2 *)(keep_cols + ((int64_t)bh * S + (kok ? kv : S - 1)) * (2 * ((S + TILE - 1) / TILE))) : nullptr;
    u32x2 keep2 = {0xffffffffu, 0xffffffffu}, keep2_next = keep2;
    if constexpr (DROP) keep2_next = keep_col[q_begin / TILE];
    for (int q0 = q_begin; q0 < S; q0 += TILE) {
        __syncthreads();
        lq.store_rows(Qs);
        ldo.store_rows(dOs);
        if constexpr (DROP) keep2 = keep2_next;
        if (threadIdx.x < TILE) {
            const int qq = q0 + threadIdx.x;
            lse_s[threadIdx.x] = qq < S ? lse_b[qq] * LOG2E : INFINITY;
            delta_s[threadIdx.x] = qq < S ? delta_b[qq] : 0.f;
        }
        __syncthreads();
        if (q0 + TILE < S) {
            const int nx = q0 + TILE;
            lq.load(Q + (int64_t)nx * ld, S - nx);
            ldo.load(dO + (int64_t)nx * E, S - nx);
            if constexpr (DROP) keep2_next = keep_col[nx / TILE];
        }
        if (blk * 128 + wave * 32 >= S) continue;                  // a wave without keys only moves tiles and meets barriers

        // one 32-row query block at a time keeps only one score / dP accumulator pair live; the loop is kept
        // rolled so that the scheduler cannot pull the second block's fragments ahead of the first one's math
#pragma unroll 1
        for (int t = 0; t < 2; ++t) {
            if (t == 1 && q0 + 32 >= S) break;                     // the sequence ends in the tile's first half: no query here
            f32x16 sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                sc = mma(frag_rowk(Qs, t * 32 + c, s, h), kf[s], sc);
                dp = mma(frag_rowk(dOs, t * 32 + c, s, h), vf[s], dp);
            }
            const uint32_t keep = t ? keep2.y : keep2.x;           // this key's 32 queries q0 + 32 t .. + 32, bit = query
            if constexpr (DROP) {
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        dp[g * 4 + e] = (keep & (1u << (g * 8 + h * 4 + e))) ? dp[g * 4 + e] * keep_scale : 0.f;
            }
            // without a mask, query rows beyond S carry lse = +inf (p = 0); causal tiles below the diagonal of the
            // block's 128 keys need no comparison
            const bool plain = !mask && (!CAUSAL || blk * 128 + 127 <= q0);
            // accumulator registers 4 g .. 4 g + 3 are query rows ql .. ql + 3; the two paths are whole loops of their
            // own (a branch per group makes the compiler copy both accumulator tiles at every merge)
            if (plain) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ql = t * 32 + g * 8 + h * 4;
                    const f32x4 l4 = *(const f32x4 *)(lse_s + ql), d4 = *(const f32x4 *)(delta_s + ql);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = g * 4 + e;
                        const float p = __builtin_amdgcn_exp2f(fmaf(sc[r], sl2, -l4[e]));
                        sc[r] = p;
                        dp[r] = p * (dp[r] - d4[e]);
                    }
                }
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int ql = t * 32 + g * 8 + h * 4;
                    const f32x4 l4 = *(const f32x4 *)(lse_s + ql), d4 = *(const f32x4 *)(delta_s + ql);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = g * 4 + e;
                        float x = fmaf(sc[r], sl2, -l4[e]);
                        if (mask) x += (kok && q0 + ql + e < S) ? mask[(int64_t)(q0 + ql + e) * S + kv] * LOG2E : 0.f;
                        const float p = (CAUSAL && kv > q0 + ql + e) ? 0.f : __builtin_amdgcn_exp2f(x);
                        sc[r] = p;
                        dp[r] = p * (dp[r] - d4[e]);
                    }
                }
            }
            if constexpr (DROP) {                                  // dV takes the dropped probabilities
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        sc[g * 4 + e] = (keep & (1u << (g * 8 + h * 4 + e))) ? sc[g * 4 + e] * keep_scale : 0.f;
            }
#pragma unroll
            for (int sp = 0; sp < 2; ++sp) {
                const frag_t pb = acc_to_b(sc, sp), db = acc_to_b(dp, sp);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    dvt[u] = mma(tr.frag(dOs, u * 32, t * 2 + sp), pb, dvt[u]);
                    dkt[u] = mma(tr.frag(Qs, u * 32, t * 2 + sp), db, dkt[u]);
                }
            }
        }
    }
    if (kok) {
        bf16_t *drow = dqkv + ((int64_t)b * S + kv) * ld + hh * HD;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                bf16x4 ok_, ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ok_[e] = (bf16_t)(dkt[u][g * 4 + e] * scale);
                    ov[e] = (bf16_t)dvt[u][g * 4 + e];
                }
                *(bf16x4 *)(drow + E + u * 32 + g * 8 + h * 4) = ok_;
                *(bf16x4 *)(drow + 2 * E + u * 32 + g * 8 + h * 4) = ov;
            }
    }
}

// ---------------------------------------------------------------------------------------------
// keep decisions of the probabilities' dropout, as bit words in the two orders the kernels above read them in
// ---------------------------------------------------------------------------------------------
// The decision for probability (bh, q, k) is the one F.dropout's kernel takes for element (bh * S + q) * row_len + k
// of a [b * H, S, row_len] tensor (row_len even, >= S), so the fused kernels and a materialised-probabilities path
// drop the same entries.  A wave takes 64 queries x 64 keys: lane = query computes its row's 64 decisions (32 hashes),
//   keep_rows[bh][q][key tile][2]    word h, bit 16 t + 4 g + e  <->  key 64 tile + 32 t + 8 g + 4 h + e
//                                    (the accumulator register order of a lane of half h in forward and dQ),
// and a 64 x 64 bit transpose across the lanes (six exchange steps) turns rows into columns: lane = key gets
//   keep_cols[bh][k][2 * query tile + w]   bit i  <->  query 64 tile + 32 w + i.
// Rows / columns beyond S are not written (keep_rows) or hold zeros for the missing queries (keep_cols).
__global__ __launch_bounds__(256) void attn_keep_bits_kernel(uint32_t *keep_rows, uint32_t *keep_cols, int S, int64_t row_len,
                                                           float p, const int64_t *state, int64_t stream_id) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const DropKey key = drop_key(state[0], state[1], stream_id, p);
    const int n_kt = (S + TILE - 1) / TILE;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kt = blockIdx.x * 4 + wave, qt = blockIdx.y;
    const int64_t bh = blockIdx.z;
    if (kt >= n_kt) return;                                        // whole waves leave; no barrier below
    const int q = qt * TILE + lane;
    uint64_t nat = 0;                                              // bit k: keep (q, key 64 kt + k)
    if (q < S) {
        const uint64_t first = (uint64_t)((bh * S + q) * row_len + (int64_t)kt * TILE);      // even
#pragma unroll 8
        for (int j = 0; j < 32; ++j) {
            const uint32_t bits = drop_pair_bits(key, (first >> 1) + j);
            nat |= (uint64_t)((bits & 0xffffU) >= key.thr) << (2 * j);
            nat |= (uint64_t)((bits >> 16) >= key.thr) << (2 * j + 1);
        }
        u32x2 w = {0u, 0u};
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                w.x |= (uint32_t)((nat >> (t * 32 + g * 8)) & 0xf) << (t * 16 + g * 4);
                w.y |= (uint32_t)((nat >> (t * 32 + g * 8 + 4)) & 0xf) << (t * 16 + g * 4);
            }
        *(u32x2 *)(keep_rows + (((int64_t)bh * S + q) * n_kt + kt) * 2) = w;
    }
    // transpose: after the step for j, bit position and lane number have exchanged their bit j
    uint64_t x = nat;
#pragma unroll
    for (int step = 0; step < 6; ++step) {
        constexpr uint64_t masks[6] = {0x00000000ffffffffull, 0x0000ffff0000ffffull, 0x00ff00ff00ff00ffull,
                                       0x0f0f0f0f0f0f0f0full, 0x3333333333333333ull, 0x5555555555555555ull};
        const int j = 32 >> step;
        const uint64_t m = masks[step];
        const uint32_t lo = __shfl_xor((uint32_t)x, j, 64), hi = __shfl_xor((uint32_t)(x >> 32), j, 64);
        const uint64_t other = ((uint64_t)hi << 32) | lo;
        x = (lane & j) ? ((x & ~m) | ((other & ~m) >> j)) : ((x & m) | ((other & m) << j));
    }
    const int k = kt * TILE + lane;
    if (k < S) {
        u32x2 w = {(uint32_t)x, (uint32_t)(x >> 32)};
        *(u32x2 *)(keep_cols + ((int64_t)bh * S + k) * (2 * n_kt) + 2 * qt) = w;
    }
}

int check_attn(const char *name, int64_t b, int64_t S, int64_t H) {
    HAPMI_REQUIRE(b >= 0 && S >= 1 && H >= 1, HAPMI_EINVAL, "%s: bad shape", name);
    HAPMI_REQUIRE(S < (1ll << 24) && b * H <= 65535, HAPMI_ELIMIT, "%s: b*H %lld above 65535 or S too long", name,
                  (long long)(b * H));
    return HAPMI_OK;
}

int attention_fwd(const char *name, const void *qkv, const float *mask, int causal, void *out, float *lse, int64_t b, int64_t S,
                  int64_t H, float scale, const uint32_t *keep_rows, float p, hipStream_t st) {
    int rc = check_attn(name, b, S, H);
    if (rc) return rc;
    if (b == 0) return HAPMI_OK;
    HAPMI_REQUIRE(qkv && out && lse, HAPMI_EINVAL, "%s: null pointer", name);
    HAPMI_REQUIRE(((uintptr_t)qkv % 16) == 0 && ((uintptr_t)out % 16) == 0 && (!mask || ((uintptr_t)mask % 16) == 0) &&
                      ((uintptr_t)keep_rows % 8) == 0,
                  HAPMI_EALIGN, "%s: pointers must be 16-byte aligned (keep words: 8)", name);
    HAPMI_REQUIRE(!(causal && mask), HAPMI_EINVAL, "%s: causal and an explicit mask exclude each other", name);
    const bf16_t *x = (const bf16_t *)qkv;
    bf16_t *o = (bf16_t *)out;
    const float *no_mask = nullptr;
    const float ks = keep_rows ? 1.0f / (1.0f - p) : 1.0f;
    dim3 grid((unsigned)hapmi_cdiv(S, 128), (unsigned)(b * H)), block(AT_THREADS);
    if (causal && keep_rows)
        hipLaunchKernelGGL((attn_fwd_kernel<true, true>), grid, block, 0, st, x, no_mask, o, lse, (int)S, (int)H, scale, keep_rows, ks);
    else if (causal)
        hipLaunchKernelGGL((attn_fwd_kernel<true, false>), grid, block, 0, st, x, no_mask, o, lse, (int)S, (int)H, scale, keep_rows, ks);
    else if (keep_rows)
        hipLaunchKernelGGL((attn_fwd_kernel<false, true>), grid, block, 0, st, x, mask, o, lse, (int)S, (int)H, scale, keep_rows, ks);
    else
        hipLaunchKernelGGL((attn_fwd_kernel<false, false>), grid, block, 0, st, x, mask, o, lse, (int)S, (int)H, scale, keep_rows, ks);
    HAPMI_CHECK_LAUNCH(name);
    return HAPMI_OK;
}

int attention_bwd(const char *name, const void *qkv, const void *out, const void *dout, const float *lse, const float *mask,
                  int causal, void *dqkv, float *delta_ws, int64_t b, int64_t S, int64_t H, float scale,
                  const uint32_t *keep_rows, const uint32_t *keep_cols, float p, hipStream_t st) {
    int rc = check_attn(name, b, S, H);
    if (rc) return rc;
    if (b == 0) return HAPMI_OK;
    HAPMI_REQUIRE(qkv && out && dout && lse && dqkv && delta_ws, HAPMI_EINVAL, "%s: null pointer", name);
    HAPMI_REQUIRE(!(causal && mask), HAPMI_EINVAL, "%s: causal and an explicit mask exclude each other", name);
    HAPMI_REQUIRE(((uintptr_t)qkv % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)dout % 16) == 0 &&
                      ((uintptr_t)dqkv % 16) == 0 && (!mask || ((uintptr_t)mask % 16) == 0) &&
                      ((uintptr_t)keep_rows % 8) == 0 && ((uintptr_t)keep_cols % 8) == 0,
                  HAPMI_EALIGN, "%s: pointers must be 16-byte aligned (keep words: 8)", name);
    const bf16_t *x = (const bf16_t *)qkv, *o = (const bf16_t *)out, *d_o = (const bf16_t *)dout;
    bf16_t *dx = (bf16_t *)dqkv;
    const float *no_mask = nullptr, *delta_in = delta_ws;
    const bool drop = keep_rows != nullptr;
    const float ks = drop ? 1.0f / (1.0f - p) : 1.0f;
    dim3 grid((unsigned)hapmi_cdiv(S, 128), (unsigned)(b * H)), block(AT_THREADS);
    if (causal && drop) {
        hipLaunchKernelGGL((attn_bwd_dq_kernel<true, true>), grid, block, 0, st, x, o, d_o, lse, delta_ws, no_mask, dx, (int)S, (int)H, scale, keep_rows, ks);
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<true, true>), grid, block, 0, st, x, d_o, lse, delta_in, no_mask, dx, (int)S, (int)H, scale, keep_cols, ks);
    } else if (causal) {
        hipLaunchKernelGGL((attn_bwd_dq_kernel<true, false>), grid, block, 0, st, x, o, d_o, lse, delta_ws, no_mask, dx, (int)S, (int)H, scale, keep_rows, ks);
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<true, false>), grid, block, 0, st, x, d_o, lse, delta_in, no_mask, dx, (int)S, (int)H, scale, keep_cols, ks);
    } else if (drop) {
        hipLaunchKernelGGL((attn_bwd_dq_kernel<false, true>), grid, block, 0, st, x, o, d_o, lse, delta_ws, mask, dx, (int)S, (int)H, scale, keep_rows, ks);
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<false, true>), grid, block, 0, st, x, d_o, lse, delta_in, mask, dx, (int)S, (int)H, scale, keep_cols, ks);
    } else {
        hipLaunchKernelGGL((attn_bwd_dq_kernel<false, false>), grid, block, 0, st, x, o, d_o, lse, delta_ws, mask, dx, (int)S, (int)H, scale, keep_rows, ks);
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<false, false>), grid, block, 0, st, x, d_o, lse, delta_in, mask, dx, (int)S, (int)H, scale, keep_cols, ks);
    }
    HAPMI_CHECK_LAUNCH(name);
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_attention_fwd(const void *qkv, const float *mask, int causal, void *out, float *lse, int64_t b,
                                   int64_t S, int64_t H, float scale, hapmi_stream_t stream) {
    return attention_fwd("attention_fwd", qkv, mask, causal, out, lse, b, S, H, scale, nullptr, 0.f, (hipStream_t)stream);
}

extern "C" int hapmi_attention_bwd(const void *qkv, const void *out, const void *dout, const float *lse,
                                   const float *mask, int causal, void *dqkv, float *delta_ws, int64_t b, int64_t S,
                                   int64_t H, float scale, hapmi_stream_t stream) {
    return attention_bwd("attention_bwd", qkv, out, dout, lse, mask, causal, dqkv, delta_ws, b, S, H, scale, nullptr, nullptr, 0.f,
                         (hipStream_t)stream);
}

extern "C" int hapmi_attention_keep_bits(uint32_t *keep_rows, uint32_t *keep_cols, int64_t b, int64_t S, int64_t H,
                                         int64_t row_len, float p, const int64_t *rng_state_dev, int64_t stream_id,
                                         hapmi_stream_t stream) {
    int rc = check_attn("attention_keep_bits", b, S, H);
    if (rc) return rc;
    HAPMI_REQUIRE(p >= 0.f && p < 1.f && row_len >= S && row_len % 2 == 0, HAPMI_EINVAL,
                  "attention_keep_bits: p = %g must lie in [0, 1) and row_len = %lld must be even and >= S", (double)p, (long long)row_len);
    if (b == 0) return HAPMI_OK;
    HAPMI_REQUIRE(keep_rows && keep_cols && rng_state_dev, HAPMI_EINVAL, "attention_keep_bits: null pointer");
    HAPMI_REQUIRE(((uintptr_t)keep_rows % 8) == 0 && ((uintptr_t)keep_cols % 8) == 0 && ((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EALIGN,
                  "attention_keep_bits: pointers must be 8-byte aligned");
    const int64_t n_kt = hapmi_cdiv(S, TILE);
    HAPMI_REQUIRE(n_kt <= 65535, HAPMI_ELIMIT, "attention_keep_bits: S too long");
    dim3 grid((unsigned)hapmi_cdiv(n_kt, 4), (unsigned)n_kt, (unsigned)(b * H));
    hipLaunchKernelGGL(attn_keep_bits_kernel, grid, dim3(256), 0, (hipStream_t)stream, keep_rows, keep_cols, (int)S, row_len, p,
                       rng_state_dev, stream_id);
    HAPMI_CHECK_LAUNCH("attention_keep_bits");
    return HAPMI_OK;
}

extern "C" int hapmi_attention_fwd_dropout(const void *qkv, const float *mask, int causal, void *out, float *lse, int64_t b,
                                           int64_t S, int64_t H, float scale, const uint32_t *keep_rows, float p,
                                           hapmi_stream_t stream) {
    HAPMI_REQUIRE(keep_rows || b == 0, HAPMI_EINVAL, "attention_fwd_dropout: null keep words");
    HAPMI_REQUIRE(p >= 0.f && p < 1.f, HAPMI_EINVAL, "attention_fwd_dropout: p = %g must lie in [0, 1)", (double)p);
    return attention_fwd("attention_fwd_dropout", qkv, mask, causal, out, lse, b, S, H, scale, keep_rows, p, (hipStream_t)stream);
}

extern "C" int hapmi_attention_bwd_dropout(const void *qkv, const void *out, const void *dout, const float *lse,
                                           const float *mask, int causal, void *dqkv, float *delta_ws, int64_t b, int64_t S,
                                           int64_t H, float scale, const uint32_t *keep_rows, const uint32_t *keep_cols, float p,
                                           hapmi_stream_t stream) {
    HAPMI_REQUIRE((keep_rows && keep_cols) || b == 0, HAPMI_EINVAL, "attention_bwd_dropout: null keep words");
    HAPMI_REQUIRE(p >= 0.f && p < 1.f, HAPMI_EINVAL, "attention_bwd_dropout: p = %g must lie in [0, 1)", (double)p);
    return attention_bwd("attention_bwd_dropout", qkv, out, dout, lse, mask, causal, dqkv, delta_ws, b, S, H, scale, keep_rows, keep_cols, p,
                         (hipStream_t)stream);
}
