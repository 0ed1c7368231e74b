// 128-bit content key of a sparsity pattern (indices + indptr), computed in one
// pass over the two arrays.  Callers use it to recognise a pattern they have
// analysed before when it arrives in different tensors (a clone, the result of
// the same symbolic product computed again), so that plans derived from the
// structure alone can be reused.
//
// key = (sum_k m(a_k + S1 * (k + 1)),  sum_k m(~a_k + S2 * (k + 1)))  mod 2^64, where a is
// the concatenation of indices, nnz, indptr, and m is a 64-bit finaliser with full
// avalanche.  Every term depends on the element and on its position, and the sum
// is commutative, so the grid may add the terms in any order.
#include "nm_common.hpp"

namespace {

using nm::kWave;

constexpr int kBlock = 256;
constexpr int kMaxBlocks = 2048;

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z ^= z >> 30;
    z *= 0xbf58476d1ce4e5b9ull;
    z ^= z >> 27;
    z *= 0x94d049bb133111ebull;
    z ^= z >> 31;
    return z;
}

__device__ __forceinline__ void add_term(uint64_t v, uint64_t pos, uint64_t &h0, uint64_t &h1) {
    h0 += mix64(v + 0x9e3779b97f4a7c15ull * (pos + 1));
    h1 += mix64(~v + 0xc2b2ae3d27d4eb4full * (pos + 1));
}

__global__ __launch_bounds__(kBlock) void hash_partial_kernel(int64_t nnz, int64_t nptr,
                                                              const int64_t *__restrict__ indices,
                                                              const int64_t *__restrict__ indptr,
                                                              uint64_t *__restrict__ partial) {
    __shared__ uint64_t s_part[2 * (kBlock / kWave)];
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    uint64_t h0 = 0, h1 = 0;
    for (int64_t k = tid; k < nnz; k += stride) add_term((uint64_t)indices[k], (uint64_t)k, h0, h1);
    for (int64_t i = tid; i < nptr; i += stride) add_term((uint64_t)indptr[i], (uint64_t)(nnz + 1 + i), h0, h1);
    if (tid == 0) add_term((uint64_t)nnz, (uint64_t)nnz, h0, h1);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        h0 += __shfl_xor(h0, off, kWave);
        h1 += __shfl_xor(h1, off, kWave);
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
        s_part[2 * wave] = h0;
        s_part[2 * wave + 1] = h1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint64_t a = 0, b = 0;
        for (int w = 0; w < kBlock / kWave; ++w) {
            a += s_part[2 * w];
            b += s_part[2 * w + 1];
        }
        partial[2 * blockIdx.x] = a;
        partial[2 * blockIdx.x + 1] = b;
    }
}

// Adds the per-workgroup parts; leaves the key in `out` (device) and, when a landing place in
// pinned host memory is given, there as well, followed by the ticket the host polls for.
__global__ __launch_bounds__(kBlock) void hash_final_kernel(int nparts, const uint64_t *__restrict__ partial,
                                                            uint64_t *__restrict__ out,
                                                            volatile uint64_t *host_landing, uint64_t ticket) {
    __shared__ uint64_t s_part[2 * (kBlock / kWave)];
    uint64_t h0 = 0, h1 = 0;
    for (int i = threadIdx.x; i < nparts; i += kBlock) {
        h0 += partial[2 * i];
        h1 += partial[2 * i + 1];
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        h0 += __shfl_xor(h0, off, kWave);
        h1 += __shfl_xor(h1, off, kWave);
    }
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) {
        s_part[2 * wave] = h0;
        s_part[2 * wave + 1] = h1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint64_t a = 0, b = 0;
        for (int w = 0; w < kBlock / kWave; ++w) {
            a += s_part[2 * w];
            b += s_part[2 * w + 1];
        }
        out[0] = a;
        out[1] = b;
        if (host_landing) {
            host_landing[0] = a;
            host_landing[1] = b;
            __threadfence_system();
            host_landing[2] = ticket;
        }
    }
}

inline int blocks_for(int64_t n) {
    int64_t g = nm::ceil_div(n > 0 ? n : 1, (int64_t)kBlock * 8);
    return (int)(g > kMaxBlocks ? kMaxBlocks : (g < 1 ? 1 : g));
}

}  // namespace

extern "C" int nm_structure_hash_bytes(size_t *bytes) {
    NM_REQUIRE(bytes != nullptr, "bytes is null");
    *bytes = (size_t)(2 * kMaxBlocks + 2) * sizeof(uint64_t);
    return NM_OK;
}

extern "C" int nm_structure_hash(int64_t nnz, int64_t nptr, const int64_t *indices, const int64_t *indptr,
                                 void *work, size_t work_bytes, void *host_landing, uint64_t *key,
                                 nm_stream stream) {
    NM_REQUIRE(nnz >= 0 && nptr >= 0 && key != nullptr, "bad arguments");
    NM_REQUIRE((nnz == 0 || indices) && (nptr == 0 || indptr) && work, "null pointer argument");
    size_t need = 0;
    nm_structure_hash_bytes(&need);
    if (work_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", work_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    uint64_t *partial = (uint64_t *)work;
    uint64_t *out = partial + 2 * kMaxBlocks;
    const int blocks = blocks_for(nnz + nptr);
    hipLaunchKernelGGL(hash_partial_kernel, dim3(blocks), dim3(kBlock), 0, s, nnz, nptr, indices, indptr, partial);
    NM_LAUNCH_CHECK("hash_partial_kernel");
    volatile uint64_t *land = (volatile uint64_t *)host_landing;
    const uint64_t ticket = land ? land[2] + 1 : 0;
    hipLaunchKernelGGL(hash_final_kernel, dim3(1), dim3(kBlock), 0, s, blocks, partial, out, land, ticket);
    NM_LAUNCH_CHECK("hash_final_kernel");
    if (land) {
        bool arrived = false;
        for (int spin = 0; spin < (1 << 22) && !arrived; ++spin) arrived = land[2] == ticket;
        if (!arrived) {
            NM_HIP_TRY(hipStreamSynchronize(s));
            NM_REQUIRE(land[2] == ticket, "the structure key did not arrive");
        }
        key[0] = land[0];
        key[1] = land[1];
        return NM_OK;
    }
    NM_HIP_TRY(hipMemcpyAsync(key, out, 2 * sizeof(uint64_t), hipMemcpyDeviceToHost, s));
    NM_HIP_TRY(hipStreamSynchronize(s));
    return NM_OK;
}

namespace {

__global__ __launch_bounds__(kBlock) void longest_row_kernel(int64_t rows, const int64_t *__restrict__ indptr,
                                                             unsigned long long *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    long long len = 0;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < rows; i += stride) {
        const long long d = indptr[i + 1] - indptr[i];
        len = d > len ? d : len;
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const long long o = __shfl_xor(len, off, kWave);
        len = o > len ? o : len;
    }
    if ((threadIdx.x & (kWave - 1)) == 0 && len > 0) atomicMax(out, (unsigned long long)len);
}

__global__ void land_word_kernel(const unsigned long long *__restrict__ word, volatile uint64_t *host_landing,
                                 uint64_t ticket) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        host_landing[0] = *word;
        __threadfence_system();
        host_landing[2] = ticket;
    }
}

}  // namespace

extern "C" int nm_csr_longest_row(int64_t rows, const int64_t *indptr, void *work, size_t work_bytes,
                                  void *host_landing, int64_t *longest, nm_stream stream) {
    NM_REQUIRE(rows >= 0 && longest != nullptr && work != nullptr && work_bytes >= 8, "bad arguments");
    NM_REQUIRE(rows == 0 || indptr != nullptr, "indptr is null");
    hipStream_t s = nm::as_stream(stream);
    unsigned long long *out = (unsigned long long *)work;
    if (int rc = nm::fill_async(out, (int64_t)1, 0ull, s)) return rc;
    if (rows > 0) {
        hipLaunchKernelGGL(longest_row_kernel, dim3(blocks_for(rows)), dim3(kBlock), 0, s, rows, indptr, out);
        NM_LAUNCH_CHECK("longest_row_kernel");
    }
    volatile uint64_t *land = (volatile uint64_t *)host_landing;
    if (land) {
        const uint64_t ticket = land[2] + 1;
        hipLaunchKernelGGL(land_word_kernel, dim3(1), dim3(64), 0, s, out, land, ticket);
        NM_LAUNCH_CHECK("land_word_kernel");
        bool arrived = false;
        for (int spin = 0; spin < (1 << 22) && !arrived; ++spin) arrived = land[2] == ticket;
        if (!arrived) {
            NM_HIP_TRY(hipStreamSynchronize(s));
            NM_REQUIRE(land[2] == ticket, "the result did not arrive");
        }
        *longest = (int64_t)land[0];
        return NM_OK;
    }
    unsigned long long host = 0;
    NM_HIP_TRY(hipMemcpyAsync(&host, out, sizeof(host), hipMemcpyDeviceToHost, s));
    NM_HIP_TRY(hipStreamSynchronize(s));
    *longest = (int64_t)host;
    return NM_OK;
}
