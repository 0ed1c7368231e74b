// In-place exclusive prefix sum of an int64 device array (three launches:
// per-block sums, scan of the sums by one workgroup, apply; one launch for short arrays).
#pragma once

#include "nm_common.hpp"

namespace nm {

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;                          // consecutive items per lane
constexpr int kScanTile = kScanBlock * kScanItems;     // items per workgroup

// Bytes of scratch scan_exclusive_i64 needs for n items.
inline size_t scan_scratch_bytes(int64_t n) {
    return (size_t)(ceil_div(n > 0 ? n : 1, kScanTile) + 1) * sizeof(int64_t);
}

// Exclusive scan over the workgroup's lanes; returns the lane's prefix and the
// workgroup total in `total`.  `s_wave` holds one slot per wavefront.
__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t *s_wave, int64_t &total) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int nwaves = blockDim.x / kWave;
    int64_t inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int64_t up = __shfl_up(inc, off, kWave);
        if (lane >= off) inc += up;
    }
    if (lane == kWave - 1) s_wave[wave] = inc;
    __syncthreads();
    int64_t before = 0;
    total = 0;
    for (int w = 0; w < nwaves; ++w) {
        const int64_t t = s_wave[w];
        if (w < wave) before += t;
        total += t;
    }
    __syncthreads();
    return before + inc - v;
}

// Whether this workgroup's tile lies inside a[0, n) whole and a's 16-byte pairs are aligned
// (uniform over the workgroup).
typedef int64_t I64x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ bool scan_tile_whole(const int64_t *a, int64_t n) {
    static_assert(kScanItems % 2 == 0, "items are loaded in pairs");
    return ((int64_t)blockIdx.x + 1) * kScanTile <= n && (reinterpret_cast<uintptr_t>(a) & 15) == 0;
}

static __global__ __launch_bounds__(kScanBlock) void scan_tile_sums_kernel(const int64_t *__restrict__ a, int64_t n,
                                                                    int64_t *__restrict__ sums) {
    __shared__ int64_t s_wave[kScanBlock / kWave];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int64_t v = 0;
    if (scan_tile_whole(a, n)) {
        // a whole tile: the lane's 64 bytes in four 16-byte loads, no test per item
        const I64x2 *p = reinterpret_cast<const I64x2 *>(a + base);
#pragma unroll
        for (int i = 0; i < kScanItems / 2; ++i) {
            const I64x2 w = p[i];
            v += w[0] + w[1];
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanItems; ++i)
            if (base + i < n) v += a[base + i];
    }
    int64_t total;
    block_exclusive_scan(v, s_wave, total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// Exclusive scan of sums[0, m) in place by one workgroup; sums[m] = grand total.
static __global__ __launch_bounds__(1024) void scan_sums_kernel(int64_t *sums, int64_t m) {
    __shared__ int64_t s_wave[1024 / kWave];
    int64_t carry = 0;
    for (int64_t c0 = 0; c0 < m; c0 += 1024) {
        const int64_t i = c0 + threadIdx.x;
        const int64_t v = i < m ? sums[i] : 0;
        int64_t total;
        const int64_t pre = block_exclusive_scan(v, s_wave, total);
        if (i < m) sums[i] = carry + pre;
        carry += total;
    }
    if (threadIdx.x == 0) sums[m] = carry;
}

static __global__ __launch_bounds__(kScanBlock) void scan_apply_kernel(int64_t *__restrict__ a, int64_t n,
                                                                const int64_t *__restrict__ sums) {
    __shared__ int64_t s_wave[kScanBlock / kWave];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int64_t item[kScanItems];
    int64_t v = 0;
    const bool whole = scan_tile_whole(a, n);
    if (whole) {
        const I64x2 *p = reinterpret_cast<const I64x2 *>(a + base);
#pragma unroll
        for (int i = 0; i < kScanItems / 2; ++i) {
            const I64x2 w = p[i];
            item[2 * i] = w[0];
            item[2 * i + 1] = w[1];
            v += w[0] + w[1];
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            item[i] = base + i < n ? a[base + i] : 0;
            v += item[i];
        }
    }
    int64_t total;
    int64_t run = sums[blockIdx.x] + block_exclusive_scan(v, s_wave, total);
    if (whole) {
        I64x2 *p = reinterpret_cast<I64x2 *>(a + base);
#pragma unroll
        for (int i = 0; i < kScanItems / 2; ++i) {
            I64x2 w;
            w[0] = run;
            w[1] = run + item[2 * i];
            run = w[1] + item[2 * i + 1];
            p[i] = w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            if (base + i < n) a[base + i] = run;
            run += item[i];
        }
    }
}

// The whole scan by one workgroup, for arrays short enough that three launches would cost more
// than the work: 8 consecutive items per lane and pass.
constexpr int kScanSmall = 8192;
static __global__ __launch_bounds__(1024) void scan_small_kernel(int64_t *a, int64_t n) {
    __shared__ int64_t s_wave[1024 / kWave];
    int64_t carry = 0;
    for (int64_t c0 = 0; c0 < n; c0 += 1024 * kScanItems) {
        const int64_t base = c0 + (int64_t)threadIdx.x * kScanItems;
        int64_t item[kScanItems];
        int64_t v = 0;
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            item[i] = base + i < n ? a[base + i] : 0;
            v += item[i];
        }
        int64_t total;
        int64_t run = carry + block_exclusive_scan(v, s_wave, total);
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            if (base + i < n) a[base + i] = run;
            run += item[i];
        }
        carry += total;
    }
}

// a[i] <- sum of a[0, i) for i in [0, n).  `scratch` holds scan_scratch_bytes(n).
inline int scan_exclusive_i64(int64_t *a, int64_t n, int64_t *scratch, hipStream_t s) {
    if (n <= 0) return NM_OK;
    if (n <= kScanSmall) {
        hipLaunchKernelGGL(scan_small_kernel, dim3(1), dim3(1024), 0, s, a, n);
        NM_LAUNCH_CHECK("scan_small_kernel");
        return NM_OK;
    }
    const int64_t tiles = ceil_div(n, kScanTile);
    if (tiles > kMaxGrid) return fail(NM_ERR_UNSUPPORTED, "scan of %lld items is too long", (long long)n);
    hipLaunchKernelGGL(scan_tile_sums_kernel, dim3((unsigned)tiles), dim3(kScanBlock), 0, s, a, n, scratch);
    NM_LAUNCH_CHECK("scan_tile_sums_kernel");
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(1024), 0, s, scratch, tiles);
    NM_LAUNCH_CHECK("scan_sums_kernel");
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)tiles), dim3(kScanBlock), 0, s, a, n, scratch);
    NM_LAUNCH_CHECK("scan_apply_kernel");
    return NM_OK;
}

}  // namespace nm
