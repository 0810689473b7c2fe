// Device-wide exclusive prefix sum used by the compaction and intersection code.
//
// Per-block totals, then a per-block scan that adds the block's base; the base comes from a
// single-workgroup scan of the totals in between or, for up to two million elements, is added
// up by every block itself (two launches instead of three).  2048 items per workgroup of 256 lanes;
// wave64 shuffles inside a wavefront, LDS across the four wavefronts.
#pragma once

#include "common.h"

#ifdef __HIPCC__

#define SCAN_ITEMS 8
#define SCAN_TILE (SPLATAD_THREADS * SCAN_ITEMS)

namespace { // one private copy of the kernels per translation unit

// How logical element i of a scan maps to memory.  stride > 0: element i sits at i * stride.
// stride < 0: the data is a [-stride][n / -stride] matrix scanned column by column, i.e.
// logical i = col * rows + row sits at row * cols + col.
__device__ __forceinline__ int64_t scan_phys(int64_t i, int64_t n, int stride) {
    if (stride > 0) return i * stride;
    const int64_t rows = -stride, cols = n / rows;
    return (i % rows) * cols + (i / rows);
}

// Walks consecutive logical elements from i on: one division at the start (n < 2^32), an
// addition per step.
struct ScanCursor {
    int64_t phys;
    uint32_t row, rows, cols;
    __device__ __forceinline__ ScanCursor(int64_t i, int64_t n, int stride) {
        if (stride > 0) {
            rows = 0; cols = (uint32_t)stride; row = 0;
            phys = i * stride;
        } else {
            rows = (uint32_t)-stride;
            cols = (uint32_t)n / rows;
            const uint32_t col = (uint32_t)i / rows;
            row = (uint32_t)i - col * rows;
            phys = (int64_t)row * cols + col;
        }
    }
    __device__ __forceinline__ void next() {
        phys += cols; // the next row of the column, or the next element of a strided vector
        if (rows != 0 && ++row == rows) {
            row = 0;
            phys -= (int64_t)rows * cols - 1; // top of the next column
        }
    }
};

// Value at a physical position, optionally reduced to a 0/1 flag (v > 0).
__device__ __forceinline__ int32_t scan_load(const int32_t *in, const ScanCursor &c, bool valid, int as_flag) {
    if (!valid) return 0;
    const int32_t v = in[c.phys];
    return as_flag ? (v > 0 ? 1 : 0) : v;
}

// Exclusive scan of one int64 per lane across the workgroup; returns the lane's
// exclusive prefix and the workgroup total.
__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t *total) {
    __shared__ int64_t wave_tot[SPLATAD_THREADS / SPLATAD_WAVE];
    const int lane = threadIdx.x & (SPLATAD_WAVE - 1);
    const int wave = threadIdx.x / SPLATAD_WAVE;
    int64_t incl = v;
#pragma unroll
    for (int off = 1; off < SPLATAD_WAVE; off <<= 1) {
        int64_t o = __shfl_up(incl, off, SPLATAD_WAVE);
        if (lane >= off) incl += o;
    }
    if (lane == SPLATAD_WAVE - 1) wave_tot[wave] = incl;
    __syncthreads();
    int64_t base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < SPLATAD_THREADS / SPLATAD_WAVE; ++w) {
        int64_t t = wave_tot[w];
        if (w < wave) base += t;
        tot += t;
    }
    __syncthreads();
    *total = tot;
    return base + incl - v;
}

__global__ void __launch_bounds__(SPLATAD_THREADS)
scan_block_totals_kernel(const int32_t *__restrict__ in, int64_t n, int stride, int as_flag,
                         int64_t *__restrict__ block_sums) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    int64_t s = 0;
    ScanCursor c(base, n, stride);
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; ++k) {
        s += scan_load(in, c, base + k < n, as_flag);
        c.next();
    }
    int64_t tot;
    block_exclusive_scan(s, &tot);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = tot;
}

// One workgroup: in-place exclusive scan of block_sums, grand total to *total.
__global__ void __launch_bounds__(SPLATAD_THREADS)
scan_block_sums_kernel(int64_t *__restrict__ block_sums, int64_t n_blocks,
                       int64_t *__restrict__ total) {
    int64_t carry = 0;
    for (int64_t start = 0; start < n_blocks; start += SPLATAD_THREADS) {
        int64_t i = start + threadIdx.x;
        int64_t v = i < n_blocks ? block_sums[i] : 0;
        int64_t tot;
        int64_t ex = block_exclusive_scan(v, &tot);
        if (i < n_blocks) block_sums[i] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) *total = carry;
}

// FOLD: block_sums holds the blocks' totals, not yet scanned; every workgroup adds up the
// totals before its own (a few hundred at most, see kScanFoldBlocks) and the last one writes
// the grand total, which saves the launch of scan_block_sums_kernel.
// fold_ratio > 1: block_sums holds that many finer totals per block (those of consecutive,
// equally long parts of it).
template <typename OutT, bool FOLD>
__global__ void __launch_bounds__(SPLATAD_THREADS)
scan_apply_kernel(const int32_t *__restrict__ in, int64_t n, int stride, int as_flag,
                  const int64_t *__restrict__ block_sums, OutT *__restrict__ out,
                  int64_t *__restrict__ total, uint32_t fold_ratio) {
    int64_t before = 0;
    if (FOLD) {
        int64_t part = 0;
        const uint32_t parts_before = blockIdx.x * fold_ratio;
        for (uint32_t j = threadIdx.x; j < parts_before; j += SPLATAD_THREADS) part += block_sums[j];
        block_exclusive_scan(part, &before);
    } else {
        before = block_sums[blockIdx.x];
    }
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    int32_t v[SCAN_ITEMS];
    int64_t s = 0;
    ScanCursor c(base, n, stride);
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; ++k) {
        v[k] = scan_load(in, c, base + k < n, as_flag);
        s += v[k];
        c.next();
    }
    int64_t tot;
    int64_t run = block_exclusive_scan(s, &tot) + before;
    if (FOLD && blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *total = before + tot;
    // the output is dense for a strided input and shares the layout of a transposed one
    ScanCursor o(base, n, stride > 0 ? 1 : stride);
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; ++k) {
        if (base + k < n) out[o.phys] = (OutT)run;
        run += v[k];
        o.next();
    }
}

constexpr int64_t kScanFoldBlocks = 1024; // up to 2M elements: two launches instead of three

// One launch for a consumer that finishes the scan itself: out holds every element's exclusive
// prefix inside its block of SCAN_TILE logical elements, block_sums the blocks' totals; the
// prefix of element i is out[phys(i)] + the sum of block_sums[0 .. i / SCAN_TILE).  For tables
// of up to kScanLocalBlocks blocks, two per lane of a consumer's wavefront, which adds them up
// with shuffles.
constexpr int64_t kScanLocalBlocks = 2 * SPLATAD_WAVE;

template <typename OutT>
__global__ void __launch_bounds__(SPLATAD_THREADS)
scan_local_kernel(const int32_t *__restrict__ in, int64_t n, int stride, OutT *__restrict__ out,
                  int64_t *__restrict__ block_sums) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    int32_t v[SCAN_ITEMS];
    int64_t s = 0;
    ScanCursor c(base, n, stride);
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; ++k) {
        v[k] = scan_load(in, c, base + k < n, 0);
        s += v[k];
        c.next();
    }
    int64_t tot;
    int64_t run = block_exclusive_scan(s, &tot);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = tot;
    ScanCursor o(base, n, stride > 0 ? 1 : stride);
#pragma unroll
    for (int k = 0; k < SCAN_ITEMS; ++k) {
        if (base + k < n) out[o.phys] = (OutT)run;
        run += v[k];
        o.next();
    }
}

static inline size_t scan_workspace_bytes(int64_t n) {
    int64_t n_blocks = (n + SCAN_TILE - 1) / SCAN_TILE;
    return splatad_align256((size_t)(n_blocks > 0 ? n_blocks : 1) * sizeof(int64_t));
}

// out[i] = sum_{j<i} f(in[phys(j)]); *total (device) = sum over all.  The output is dense for
// stride > 0 and uses the input's transposed layout for stride < 0 (see scan_phys).
// `block_sums` is scan_workspace_bytes(n) of scratch.  n == 0 only writes *total = 0.
// Second half of a scan whose per-block totals (SCAN_TILE logical elements per block) are in
// block_sums already: launch_exclusive_scan() below, or a caller that makes the totals with a
// kernel of its own, which can gather something else on the same pass.
template <typename OutT>
static inline int launch_exclusive_scan_apply(const int32_t *in, int64_t n, int stride, int as_flag,
                                              OutT *out, int64_t *total, int64_t *block_sums,
                                              hipStream_t stream, uint32_t fold_ratio = 1) {
    const int64_t n_blocks = (n + SCAN_TILE - 1) / SCAN_TILE;
    if (n_blocks > 0 && n_blocks <= kScanFoldBlocks && out != nullptr) {
        hipLaunchKernelGGL((scan_apply_kernel<OutT, true>), dim3((uint32_t)n_blocks),
                           dim3(SPLATAD_THREADS), 0, stream, in, n, stride, as_flag,
                           (const int64_t *)block_sums, out, total, fold_ratio);
        SPLATAD_LAUNCH_CHECK();
        return 0;
    }
    SPLATAD_REQUIRE(fold_ratio == 1, "scan: finer totals need the folding pass (%lld blocks)", (long long)n_blocks);
    hipLaunchKernelGGL(scan_block_sums_kernel, dim3(1), dim3(SPLATAD_THREADS), 0, stream,
                       block_sums, n_blocks, total);
    SPLATAD_LAUNCH_CHECK();
    if (n_blocks > 0 && out != nullptr) {
        hipLaunchKernelGGL((scan_apply_kernel<OutT, false>), dim3((uint32_t)n_blocks),
                           dim3(SPLATAD_THREADS), 0, stream, in, n, stride, as_flag,
                           (const int64_t *)block_sums, out, total, 1u);
        SPLATAD_LAUNCH_CHECK();
    }
    return 0;
}

// Returns the number of blocks through *n_blocks; the caller has checked n against
// kScanLocalBlocks * SCAN_TILE.
template <typename OutT>
static inline int launch_local_scan(const int32_t *in, int64_t n, int stride, OutT *out,
                                    int64_t *block_sums, uint32_t *n_blocks, hipStream_t stream) {
    const int64_t blocks = (n + SCAN_TILE - 1) / SCAN_TILE;
    SPLATAD_REQUIRE(n > 0 && blocks <= kScanLocalBlocks, "scan: %lld elements are too many for a local scan", (long long)n);
    hipLaunchKernelGGL((scan_local_kernel<OutT>), dim3((uint32_t)blocks), dim3(SPLATAD_THREADS), 0, stream, in, n,
                       stride, out, block_sums);
    SPLATAD_LAUNCH_CHECK();
    *n_blocks = (uint32_t)blocks;
    return 0;
}

template <typename OutT>
static inline int launch_exclusive_scan(const int32_t *in, int64_t n, int stride, int as_flag,
                                        OutT *out, int64_t *total, int64_t *block_sums,
                                        hipStream_t stream) {
    SPLATAD_REQUIRE(n >= 0 && n < ((int64_t)1 << 32), "scan: %lld elements exceed the 32-bit index range", (long long)n);
    const int64_t n_blocks = (n + SCAN_TILE - 1) / SCAN_TILE;
    if (n_blocks > 0) {
        hipLaunchKernelGGL(scan_block_totals_kernel, dim3((uint32_t)n_blocks), dim3(SPLATAD_THREADS),
                           0, stream, in, n, stride, as_flag, block_sums);
        SPLATAD_LAUNCH_CHECK();
    }
    return launch_exclusive_scan_apply<OutT>(in, n, stride, as_flag, out, total, block_sums, stream);
}

} // namespace

#endif // __HIPCC__
