// Counter-based keep / drop decisions for F.dropout in training mode.
//
// The decision for an element is a pure function of (seed, step, stream id, element index): no generator state
// is carried between elements, so forward and backward of one node regenerate the same mask from the same four
// numbers instead of storing it, any kernel can apply the mask to the elements it happens to hold, and a step
// replayed from a HIP graph takes a fresh mask because `step` lives in device memory and is advanced by a kernel.
// seed and step are the two int64 of the RNG state; the stream id names the dropout node inside a program.
//
// One 32-bit hash serves two neighbouring elements (its halves are compared with p * 65536), so p is realised to
// within 2^-17.  The hash is two rounds of multiply-xorshift mixing per element pair.
#pragma once
#include <stdint.h>

struct DropKey {
    uint32_t k0, k1;       // per (seed, step, stream id)
    uint32_t thr;          // an element is kept iff its 16 random bits are >= thr
    float scale;           // 1 / (1 - p)
};

__host__ __device__ __forceinline__ uint32_t drop_mix32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

__host__ __device__ __forceinline__ DropKey drop_key(int64_t seed, int64_t step, int64_t stream_id, float p) {
    uint32_t k = drop_mix32((uint32_t)(uint64_t)seed ^ 0x9e3779b9U);
    k = drop_mix32(k ^ (uint32_t)((uint64_t)seed >> 32));
    k = drop_mix32(k ^ (uint32_t)(uint64_t)step);
    k = drop_mix32(k ^ (uint32_t)((uint64_t)step >> 32) ^ 0x85ebca6bU);
    k = drop_mix32(k ^ (uint32_t)(uint64_t)stream_id);
    DropKey key;
    key.k0 = k;
    key.k1 = drop_mix32(k ^ 0xc2b2ae35U ^ (uint32_t)((uint64_t)stream_id >> 32));
    float t = p * 65536.0f + 0.5f;
    key.thr = t <= 0.f ? 0u : (t >= 65536.0f ? 65536u : (uint32_t)t);
    key.scale = p < 1.0f ? 1.0f / (1.0f - p) : 0.0f;
    return key;
}

// 32 random bits for the element pair (2 j, 2 j + 1): low half for the even element, high half for the odd one
__host__ __device__ __forceinline__ uint32_t drop_pair_bits(const DropKey &key, uint64_t j) {
    return drop_mix32(drop_mix32((uint32_t)j + key.k0) ^ ((uint32_t)(j >> 32) * 0x9e3779b9U + key.k1));
}

__host__ __device__ __forceinline__ bool drop_keep(const DropKey &key, uint64_t index) {
    const uint32_t r = drop_pair_bits(key, index >> 1);
    return ((index & 1) ? (r >> 16) : (r & 0xffffU)) >= key.thr;
}
