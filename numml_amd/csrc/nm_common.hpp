// Shared host/device helpers of libnumml_hip.so (gfx950 only).
#pragma once
#include <utility>

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "numml_hip.h"

namespace nm {

constexpr int kWave = 64;  // CDNA wavefront width

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char *fmt, ...);

#define NM_HIP_TRY(expr)                                                          \
    do {                                                                          \
        hipError_t nm_e_ = (expr);                                                \
        if (nm_e_ != hipSuccess)                                                  \
            return ::nm::fail(NM_ERR_HIP, "%s failed: %s (%s:%d)", #expr,         \
                              hipGetErrorString(nm_e_), __FILE__, __LINE__);      \
    } while (0)

// Checks the launch that was just enqueued.
#define NM_LAUNCH_CHECK(name)                                                     \
    do {                                                                          \
        hipError_t nm_e_ = hipGetLastError();                                     \
        if (nm_e_ != hipSuccess)                                                  \
            return ::nm::fail(NM_ERR_HIP, "launch of %s failed: %s", name,        \
                              hipGetErrorString(nm_e_));                          \
    } while (0)

#define NM_REQUIRE(cond, ...)                                                     \
    do {                                                                          \
        if (!(cond)) return ::nm::fail(NM_ERR_INVALID, __VA_ARGS__);              \
    } while (0)

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Grid sizes are 32-bit in HIP; every launcher caps its 1-D grid below this
// and the kernels stride.
constexpr int64_t kMaxGrid = 1 << 30;

// MI355X has 8 accelerator dies (XCDs), each with a private L2; the hardware
// deals consecutive workgroup ids round-robin over them.  xcd_tile() turns the
// workgroup id into a tile index such that every XCD walks one contiguous
// eighth of the tiles, which keeps cache lines shared by neighbouring tiles
// (halo reads, partially written lines) inside one L2.  `ntiles_padded` is
// xcd_padded(ntiles); ids that map past `ntiles` own no tile.
constexpr int kXcds = 8;
__host__ __device__ inline int64_t xcd_padded(int64_t ntiles) { return (ntiles + kXcds - 1) / kXcds * kXcds; }
__device__ __forceinline__ int64_t xcd_tile(int64_t id, int64_t ntiles_padded) {
    const int64_t per = ntiles_padded / kXcds;
    return (id % kXcds) * per + id / kXcds;
}

// Same dealing, but every XCD walks its eighth from the far end: a backward pass
// that follows a forward pass then starts on the data the forward touched last,
// which is what the memory-side cache still holds.
__device__ __forceinline__ int64_t xcd_tile_reversed(int64_t id, int64_t ntiles_padded) {
    const int64_t per = ntiles_padded / kXcds;
    return (id % kXcds) * per + (per - 1 - id / kXcds);
}

inline hipStream_t as_stream(nm_stream s) { return reinterpret_cast<hipStream_t>(s); }

// ---- device helpers -------------------------------------------------------

// Data-parallel-primitive move: every lane reads the lane selected by CTRL
// (a DPP control word) without going through LDS; lanes in rows masked off by
// ROW_MASK receive 0.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_move(double v) {
    const long long bits = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(bits & 0xffffffffll), CTRL, ROW_MASK, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(bits >> 32), CTRL, ROW_MASK, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_move(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}

// Same move with zero fill: lanes whose source lies outside the row (shifts)
// read 0, so no previous value has to be supplied.
template <int CTRL>
__device__ __forceinline__ float dpp_move_zero(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move_zero(double v) {
    const long long bits = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)(bits & 0xffffffffll), CTRL, 0xf, 0xf, true);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(bits >> 32), CTRL, 0xf, 0xf, true);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

template <int CTRL>
__device__ __forceinline__ int dpp_move_zero(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a
// compile-time constant in the body (DPP controls, register arrays).
template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
}

// Lane N of every aligned row of 16 lanes, handed to all lanes of that row (v_mov_b32_dpp
// row_newbcast: one vector instruction per 32 bits, where a shuffle by lane number goes through
// the LDS crossbar and waits for it).
template <int N> __device__ __forceinline__ int row_lane(int v) {
    static_assert(N >= 0 && N < 16, "a lane of a row of 16");
    return __builtin_amdgcn_update_dpp(0, v, 0x150 + N, 0xf, 0xf, false);
}
template <int N> __device__ __forceinline__ int64_t row_lane(int64_t v) {
    const int lo = row_lane<N>((int)(v & 0xffffffffll)), hi = row_lane<N>((int)(v >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}
template <int N> __device__ __forceinline__ float row_lane(float v) { return __int_as_float(row_lane<N>(__float_as_int(v))); }
// Lane LO of the row to its lanes 0-7 and lane HI to its lanes 8-15 (two moves, each writing two
// of the row's four banks).
template <int LO, int HI> __device__ __forceinline__ int row_lane_halves(int v) {
    static_assert(LO >= 0 && LO < 16 && HI >= 0 && HI < 16, "lanes of a row of 16");
    const int r = __builtin_amdgcn_update_dpp(0, v, 0x150 + LO, 0xf, 0x3, false);
    return __builtin_amdgcn_update_dpp(r, v, 0x150 + HI, 0xf, 0xc, false);
}
template <int LO, int HI> __device__ __forceinline__ int64_t row_lane_halves(int64_t v) {
    const int lo = row_lane_halves<LO, HI>((int)(v & 0xffffffffll)), hi = row_lane_halves<LO, HI>((int)(v >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}
template <int N> __device__ __forceinline__ double row_lane(double v) {
    return __longlong_as_double(row_lane<N>((int64_t)__double_as_longlong(v)));
}

__device__ __forceinline__ float read_lane(float v, int l) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
__device__ __forceinline__ double read_lane(double v, int l) {
    const long long bits = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)(bits & 0xffffffffll), l);
    const int hi = __builtin_amdgcn_readlane((int)(bits >> 32), l);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ int read_lane(int v, int l) { return __builtin_amdgcn_readlane(v, l); }

// Sum over the 64 lanes of a wavefront with DPP adds (no LDS traffic); every
// lane gets the total.  Steps: swap within pairs, within quads, rotate the
// 16-lane row by 4 and 8 (row totals everywhere), then carry lane 15 into rows
// 1 and 3 and lane 31 into rows 2 and 3; lane 63 then holds the sum.
template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
    v += dpp_move<0xB1>(v);         // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);         // quad_perm [2,3,0,1]
    v += dpp_move<0x124>(v);        // row_ror 4
    v += dpp_move<0x128>(v);        // row_ror 8
    v += dpp_move<0x142, 0xa>(v);   // row_bcast 15 -> rows 1, 3
    v += dpp_move<0x143, 0xc>(v);   // row_bcast 31 -> rows 2, 3
    return read_lane(v, kWave - 1);
}

// Sum inside aligned groups of G consecutive lanes (G a power of two <= 64).
template <int G, typename T>
__device__ __forceinline__ T group_sum(T v) {
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Hardware floating-point atomic add without a returned value
// (global_atomic_add_f32 / _f64).
__device__ __forceinline__ void atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

// Streaming access: data that is read or written exactly once bypasses the
// cache retention policy (nontemporal), which leaves L2 to the gathered
// operands.  Measured on MI355X SpMV: 62 -> 54 us forward.
template <typename T> __device__ __forceinline__ T stream_load(const T *p) { return __builtin_nontemporal_load(p); }
template <typename T> __device__ __forceinline__ void stream_store(T *p, T v) { __builtin_nontemporal_store(v, p); }

// out[i] = v for i in [0, n): used instead of hipMemsetAsync so that callers
// may capture these entry points into HIP graphs.
template <typename T>
__global__ void fill_kernel(T *__restrict__ out, int64_t n, T v) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = v;
}

template <typename T>
inline int fill_async(T *out, int64_t n, T v, hipStream_t s) {
    if (n <= 0) return NM_OK;
    const int block = 256;
    int64_t grid = ceil_div(n, (int64_t)block * 4);
    if (grid > 65536) grid = 65536;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(fill_kernel<T>, dim3((unsigned)grid), dim3(block), 0, s, out, n, v);
    NM_LAUNCH_CHECK("fill_kernel");
    return NM_OK;
}

}  // namespace nm
