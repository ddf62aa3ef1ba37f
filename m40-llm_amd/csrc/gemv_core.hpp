// Batch-1 GEMV core shared by the standalone GEMV entry point and the fused decode kernels, so that
// both produce identical bits for the same (N, K).
//
// A workgroup has four waves.  KSPLIT == 1: every wave owns COLS output columns and walks the whole
// K range.  KSPLIT == 4: the four waves share COLS columns and each walks a quarter of K (used when
// there are few columns but a long K, which would otherwise leave too few bytes in flight); the four
// partial sums are added in wave order through LDS.  Within a wave, lane l multiplies 16-byte chunks
// l, l+64, ... of its range with one FMA chain per column, then the lanes are summed by a butterfly.
#pragma once

#include "common.hpp"

#ifdef __HIPCC__

constexpr int kGemvPrefetch = 4;   // 16-byte chunks per lane and column requested before any use

struct GemvShape {
    int cols;     // columns per wave (KSPLIT 1) or per workgroup (KSPLIT 4)
    int ksplit;   // 1 or 4
    int blocks;   // workgroups of 256 threads
};

// Host-side choice, identical for the standalone and the fused paths.
static inline GemvShape gemv_pick_shape(int N, int K) {
    GemvShape s;
    s.ksplit = (N < 4096 && K >= 4096) ? 4 : 1;
    if (s.ksplit == 4) {
        s.cols = 2;        // measured on the whole token: two columns per workgroup beat one and four
        s.blocks = (N + s.cols - 1) / s.cols;
    } else {
        s.cols = N >= 16384 ? 4 : (N >= 6144 ? 2 : 1);
        s.blocks = (N + 4 * s.cols - 1) / (4 * s.cols);
    }
    return s;
}

template <int COLS>
struct GemvRegs {
    uint4 w[kGemvPrefetch][COLS];
};

// chunk range of this wave
template <int KSPLIT>
__device__ __forceinline__ void gemv_range(int K, int wave, int* c_begin, int* c_end) {
    const int nch = K >> 3;
    if (KSPLIT == 1) {
        *c_begin = 0;
        *c_end = nch;
    } else {
        *c_begin = (int)(((long long)wave * nch) / KSPLIT);
        *c_end = (int)(((long long)(wave + 1) * nch) / KSPLIT);
    }
}

// Issue the first kGemvPrefetch loads of every column (before any prologue that the caller runs).  Chunks past the
// end of the range re-read the range's first chunk and are ignored later, so no load sits under a per-lane branch
// (waits count in issue order; a load that only some paths issue makes every later wait conservative).
// SKIP_EMPTY: a slot that lies past the end for the whole wave is not requested at all (a uniform branch; used where
// K is split over the waves and every load is awaited at once anyway).
template <int COLS, bool SKIP_EMPTY = false>
__device__ __forceinline__ void gemv_prefetch(const uint4* const (&bp)[COLS], int c_begin, int c_end, int lane,
                                              GemvRegs<COLS>& r) {
#pragma unroll
    for (int i = 0; i < kGemvPrefetch; ++i) {
        if (SKIP_EMPTY && c_begin + 64 * i >= c_end) break;
        int kc = c_begin + lane + 64 * i;
        kc = kc < c_end ? kc : c_begin;
#pragma unroll
        for (int c = 0; c < COLS; ++c) r.w[i][c] = m40_load_stream(bp[c] + kc);
    }
}

// Activations of the prefetched chunks, read from global memory.  Callers issue this before gemv_prefetch: loads
// return in issue order, so the activations (cache hits) are there when the first weights arrive.
struct GemvActRegs {
    float4 lo[kGemvPrefetch], hi[kGemvPrefetch];
};
__device__ __forceinline__ void gemv_prefetch_acts(const float* __restrict__ a, int c_begin, int c_end, int lane,
                                                   GemvActRegs& r) {
#pragma unroll
    for (int i = 0; i < kGemvPrefetch; ++i) {
        int kc = c_begin + lane + 64 * i;
        kc = kc < c_end ? kc : c_begin;
        r.lo[i] = *reinterpret_cast<const float4*>(a + 8 * kc);
        r.hi[i] = *reinterpret_cast<const float4*>(a + 8 * kc + 4);
    }
}

__device__ __forceinline__ void gemv_fma8(const uint4& w, const float4& a0, const float4& a1, float& acc) {
    float f[8];
    m40_unpack8(w, f);
    acc = fmaf(a0.x, f[0], acc);
    acc = fmaf(a0.y, f[1], acc);
    acc = fmaf(a0.z, f[2], acc);
    acc = fmaf(a0.w, f[3], acc);
    acc = fmaf(a1.x, f[4], acc);
    acc = fmaf(a1.y, f[5], acc);
    acc = fmaf(a1.z, f[6], acc);
    acc = fmaf(a1.w, f[7], acc);
}
__device__ __forceinline__ void gemv_fma8(const uint4& w, const float* __restrict__ a, int kc, float& acc) {
    gemv_fma8(w, *reinterpret_cast<const float4*>(a + 8 * kc), *reinterpret_cast<const float4*>(a + 8 * kc + 4), acc);
}

// Rest of the range beyond the prefetched chunks.
template <int COLS>
__device__ __forceinline__ void gemv_accumulate_tail(const uint4* const (&bp)[COLS], const float* __restrict__ a,
                                                     int c_begin, int c_end, int lane, float (&acc)[COLS]) {
#pragma unroll 2
    for (int kc = c_begin + lane + 64 * kGemvPrefetch; kc < c_end; kc += 64) {
        uint4 w[COLS];
#pragma unroll
        for (int c = 0; c < COLS; ++c) w[c] = m40_load_stream(bp[c] + kc);
#pragma unroll
        for (int c = 0; c < COLS; ++c) gemv_fma8(w[c], a, kc, acc[c]);
    }
}

// Consume the prefetched chunks, then the rest of the range.  `a` may point to global memory or LDS.
template <int COLS>
__device__ __forceinline__ void gemv_accumulate(const uint4* const (&bp)[COLS], const float* __restrict__ a,
                                                int c_begin, int c_end, int lane, const GemvRegs<COLS>& r,
                                                float (&acc)[COLS]) {
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[c] = 0.0f;
#pragma unroll
    for (int i = 0; i < kGemvPrefetch; ++i) {
        const int kc = c_begin + lane + 64 * i;
        if (kc < c_end) {
#pragma unroll
            for (int c = 0; c < COLS; ++c) gemv_fma8(r.w[i][c], a, kc, acc[c]);
        }
    }
    gemv_accumulate_tail<COLS>(bp, a, c_begin, c_end, lane, acc);
}

// The same with the activations of the prefetched chunks already in registers (same arithmetic, same order).
template <int COLS>
__device__ __forceinline__ void gemv_accumulate(const uint4* const (&bp)[COLS], const float* __restrict__ a,
                                                int c_begin, int c_end, int lane, const GemvRegs<COLS>& r,
                                                const GemvActRegs& ar, float (&acc)[COLS]) {
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[c] = 0.0f;
#pragma unroll
    for (int i = 0; i < kGemvPrefetch; ++i) {
        const int kc = c_begin + lane + 64 * i;
        if (kc < c_end) {
#pragma unroll
            for (int c = 0; c < COLS; ++c) gemv_fma8(r.w[i][c], ar.lo[i], ar.hi[i], acc[c]);
        }
    }
    gemv_accumulate_tail<COLS>(bp, a, c_begin, c_end, lane, acc);
}

// Lane butterfly, then (KSPLIT == 4) the four wave partials in wave order.  `red` is LDS of at
// least 4*COLS floats; the result is valid in every lane of wave 0 (KSPLIT 4) or of the wave itself.
template <int COLS, int KSPLIT>
__device__ __forceinline__ void gemv_finish(float (&acc)[COLS], float* red, int wave, int lane) {
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[c] = m40_sum64(acc[c]);
    if (KSPLIT > 1) {
        if (lane == 0) {
#pragma unroll
            for (int c = 0; c < COLS; ++c) red[wave * COLS + c] = acc[c];
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            float v = red[c];
#pragma unroll
            for (int w = 1; w < KSPLIT; ++w) v += red[w * COLS + c];
            acc[c] = v;
        }
    }
}

#endif  // __HIPCC__
