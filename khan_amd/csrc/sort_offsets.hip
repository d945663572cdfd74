// Integer part of the featurization path on gfx950: molecule offsets and the atom-type sort.
//
// ani_sort (reference: gpu_featurizer/ani_sort.cpp:71-115, a host std::stable_sort) is a stable
// 4-bin counting sort, i.e. four exclusive prefix sums over the atom array:
//     atom_counts[t]  = #{A == t}
//     scatter_idxs[g] = #{g' < g : A[g'] == A[g]}                       (rank inside its type)
//     gather_idxs[g]  = sum_{t < A[g]} atom_counts[t] + scatter_idxs[g]  (stable sort position)
// Three launches: per-tile histograms (wave ballot + popcount), a scan of the tile histograms, and
// a rank pass that redoes the ballots and adds lane / wave / tile prefixes.  Results are integers
// and identical to the host algorithm.
//
// mol_offsets (reference: tf.segment_sum(ones_like(m), m) and tf.cumsum(exclusive=True),
// khan/training/trainer_multi_tower.py:302-303) turns sorted per-atom molecule ids into per-molecule
// atom counts and exclusive offsets by locating the segment boundaries.
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

namespace {

constexpr int kSortThreads = 256;
constexpr int kSortSubTiles = 8;
constexpr int kSortTile = kSortThreads * kSortSubTiles;   // atoms per workgroup

// counts of each type among the 64 lanes, and this lane's rank among earlier lanes of its type
__device__ __forceinline__ void wave_type_masks(int type, bool valid, unsigned long long m[4])
{
#pragma unroll
    for (int t = 0; t < 4; ++t) m[t] = wave_ballot(valid && type == t);
}

__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(const int32_t* __restrict__ A,
                                                                  int64_t n,
                                                                  int32_t* __restrict__ tile_counts)
{
    __shared__ int32_t wave_counts[4][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kSortTile;
    int32_t cnt[4] = {0, 0, 0, 0};
    for (int s = 0; s < kSortSubTiles; ++s) {
        const int64_t g = tile0 + s * kSortThreads + threadIdx.x;
        const bool valid = g < n;
        const int type = valid ? fold_type(A[g]) : 0;
        unsigned long long m[4];
        wave_type_masks(type, valid, m);
#pragma unroll
        for (int t = 0; t < 4; ++t) cnt[t] += __popcll(m[t]);
    }
    if (lane == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) wave_counts[wave][t] = cnt[t];
    }
    __syncthreads();
    if (threadIdx.x < 4) {
        const int t = threadIdx.x;
        tile_counts[static_cast<int64_t>(blockIdx.x) * 4 + t] =
            wave_counts[0][t] + wave_counts[1][t] + wave_counts[2][t] + wave_counts[3][t];
    }
}

// Exclusive scan over tiles of the 4 per-tile counts, in place; totals[0..3] = atom_counts and
// totals[4..7] = exclusive type bases.  One workgroup; tiles are consumed 256 at a time.
__global__ __launch_bounds__(256) void sort_scan_kernel(int32_t* __restrict__ tile_counts,
                                                        int64_t n_tiles,
                                                        int32_t* __restrict__ totals,
                                                        int32_t* __restrict__ counts_out)
{
    __shared__ int32_t wave_tot[4][4];
    __shared__ int32_t carry[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x < 4) carry[threadIdx.x] = 0;
    __syncthreads();
    for (int64_t base = 0; base < n_tiles; base += 256) {
        const int64_t b = base + threadIdx.x;
        int32_t v[4] = {0, 0, 0, 0};
        if (b < n_tiles) {
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = tile_counts[b * 4 + t];
        }
        int32_t incl[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int32_t x = v[t];
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int32_t y = __shfl_up(x, d, 64);
                if (lane >= d) x += y;
            }
            incl[t] = x;
        }
        if (lane == 63) {
#pragma unroll
            for (int t = 0; t < 4; ++t) wave_tot[wave][t] = incl[t];
        }
        __syncthreads();
        int32_t prefix[4], chunk_total[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int32_t p = carry[t];
            for (int w = 0; w < wave; ++w) p += wave_tot[w][t];
            prefix[t] = p;
            chunk_total[t] = wave_tot[0][t] + wave_tot[1][t] + wave_tot[2][t] + wave_tot[3][t];
        }
        if (b < n_tiles) {
#pragma unroll
            for (int t = 0; t < 4; ++t) tile_counts[b * 4 + t] = prefix[t] + incl[t] - v[t];
        }
        __syncthreads();
        if (threadIdx.x < 4) carry[threadIdx.x] += chunk_total[threadIdx.x];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        int32_t run = 0;
        for (int t = 0; t < 4; ++t) {
            totals[t] = carry[t];
            totals[4 + t] = run;
            counts_out[t] = carry[t];
            run += carry[t];
        }
    }
}

__global__ __launch_bounds__(kSortThreads) void sort_rank_kernel(
    const int32_t* __restrict__ A, int64_t n, const int32_t* __restrict__ tile_base,
    const int32_t* __restrict__ totals, int32_t* __restrict__ scatter, int32_t* __restrict__ gather)
{
    __shared__ int32_t wave_counts[4][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kSortTile;
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int32_t running[4], type_base[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        running[t] = tile_base[static_cast<int64_t>(blockIdx.x) * 4 + t];
        type_base[t] = totals[4 + t];
    }
    for (int s = 0; s < kSortSubTiles; ++s) {
        const int64_t g = tile0 + s * kSortThreads + threadIdx.x;
        const bool valid = g < n;
        const int type = valid ? fold_type(A[g]) : 0;
        unsigned long long m[4];
        wave_type_masks(type, valid, m);
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < 4; ++t) wave_counts[wave][t] = __popcll(m[t]);
        }
        __syncthreads();
        int32_t rank = 0, tbase = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            int32_t before = running[t];
            for (int w = 0; w < wave; ++w) before += wave_counts[w][t];
            if (type == t) {
                rank = before + __popcll(m[t] & lt_mask);
                tbase = type_base[t];
            }
            running[t] += wave_counts[0][t] + wave_counts[1][t] + wave_counts[2][t] + wave_counts[3][t];
        }
        if (valid) {
            scatter[g] = rank;
            gather[g] = tbase + rank;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void mol_bounds_kernel(const int32_t* __restrict__ mol_idxs,
                                                         int64_t n, int32_t n_mols,
                                                         int32_t* __restrict__ MOs)
{
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g > n) return;
    int64_t prev = (g > 0) ? mol_idxs[g - 1] : -1;
    int64_t cur = (g < n) ? mol_idxs[g] : n_mols;
    if (cur > n_mols - 1) cur = n_mols - 1;   // also keeps ids beyond n_mols from writing out of range
    if (prev < -1) prev = -1;
    // every molecule id in (prev, cur] starts at atom g (ids skipped by the input are empty molecules)
    for (int64_t m = prev + 1; m <= cur; ++m) MOs[m] = static_cast<int32_t>(g);
}

__global__ __launch_bounds__(256) void mol_counts_kernel(const int32_t* __restrict__ MOs, int64_t n,
                                                         int32_t n_mols, int32_t* __restrict__ MACs)
{
    const int64_t m = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (m >= n_mols) return;
    const int32_t next = (m + 1 < n_mols) ? MOs[m + 1] : static_cast<int32_t>(n);
    MACs[m] = next - MOs[m];
}

__global__ void zero_counts_kernel(int32_t* counts4)
{
    if (threadIdx.x < 4) counts4[threadIdx.x] = 0;
}

// clears the class counts and cursors behind a size order (a kernel and not a memset node, so that the
// sequence can be recorded into a graph)
__global__ __launch_bounds__(kSizeOrderScratch) void size_clear_kernel(int32_t* __restrict__ scratch)
{
    scratch[threadIdx.x] = 0;
}

// zeros for outputs that no molecule covers (a kernel, not a memset node: see size_clear_kernel)
template <typename T>
__global__ __launch_bounds__(256) void zero_fill_kernel(T* __restrict__ a, int64_t n)
{
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
        a[i] = T(0);
}

}  // namespace

template <typename T>
hipError_t launch_zero(T* a, int64_t n, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    const int64_t want = (n + 255) / 256;
    zero_fill_kernel<T><<<dim3(static_cast<unsigned>(want < 8192 ? want : 8192)), dim3(256), 0, stream>>>(a, n);
    return hipGetLastError();
}
template hipError_t launch_zero<float>(float*, int64_t, hipStream_t);
template hipError_t launch_zero<double>(double*, int64_t, hipStream_t);

hipError_t launch_mol_offsets(const int32_t* mol_idxs, int64_t n_atoms, int32_t n_mols,
                              int32_t* MACs, int32_t* MOs, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const int64_t blocks_a = (n_atoms + 1 + 255) / 256;
    mol_bounds_kernel<<<dim3(static_cast<unsigned>(blocks_a)), dim3(256), 0, stream>>>(mol_idxs, n_atoms, n_mols, MOs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t blocks_m = (static_cast<int64_t>(n_mols) + 255) / 256;
    mol_counts_kernel<<<dim3(static_cast<unsigned>(blocks_m)), dim3(256), 0, stream>>>(MOs, n_atoms, n_mols, MACs);
    return hipGetLastError();
}

hipError_t launch_ani_sort(const int32_t* A, int64_t n_atoms, int32_t* scatter, int32_t* gather,
                           int32_t* counts4, hipStream_t stream)
{
    if (n_atoms <= 0) {
        zero_counts_kernel<<<dim3(1), dim3(64), 0, stream>>>(counts4);
        return hipGetLastError();
    }
    const int64_t n_tiles = (n_atoms + kSortTile - 1) / kSortTile;
    int32_t* ws = nullptr;   // [n_tiles*4] tile counts -> tile bases, then [8] totals and type bases
    hipError_t e = hipMallocAsync(reinterpret_cast<void**>(&ws), sizeof(int32_t) * (n_tiles * 4 + 8), stream);
    if (e != hipSuccess) return e;
    int32_t* totals = ws + n_tiles * 4;
    sort_hist_kernel<<<dim3(static_cast<unsigned>(n_tiles)), dim3(kSortThreads), 0, stream>>>(A, n_atoms, ws);
    sort_scan_kernel<<<dim3(1), dim3(256), 0, stream>>>(ws, n_tiles, totals, counts4);
    sort_rank_kernel<<<dim3(static_cast<unsigned>(n_tiles)), dim3(kSortThreads), 0, stream>>>(A, n_atoms, ws, totals, scatter, gather);
    e = hipGetLastError();
    const hipError_t e2 = hipFreeAsync(ws, stream);
    return (e != hipSuccess) ? e : e2;
}

// ---- molecules in order of decreasing atom count ----
// Counting sort of the molecule indices by min(atom count, 257), largest first.  Two passes over the
// molecules, 1,024 per workgroup: the first adds workgroup histograms (LDS integer atomics) into a global
// one; the second recomputes its histogram, reserves a range per size class with one global atomic, and
// places its molecules inside the ranges.  The order inside a size class is whatever the atomics give,
// which no result depends on.  The one-wavefront kernels take molecule order[b] in workgroup b (the
// workgroup-per-molecule kernels walk the same order with the grid's stride): the dispatcher hands out
// workgroups in index order, so the expensive molecules start first and a launch does not end on a few
// long waves.
namespace {
constexpr int kOrderThreads = 1024;

__global__ __launch_bounds__(kOrderThreads) void size_hist_kernel(const int32_t* __restrict__ MACs, int32_t n_mols,
                                                                   int32_t* __restrict__ ghist)
{
    __shared__ int hist[kSizeBins];
    const int tid = threadIdx.x;
    if (tid < kSizeBins) hist[tid] = 0;
    __syncthreads();
    const int m = blockIdx.x * kOrderThreads + tid;
    if (m < n_mols) atomicAdd(&hist[size_bin(MACs[m])], 1);
    __syncthreads();
    if (tid < kSizeBins && hist[tid] > 0) atomicAdd(&ghist[tid], hist[tid]);
}

__global__ __launch_bounds__(kOrderThreads) void size_place_kernel(const int32_t* __restrict__ MACs, int32_t n_mols,
                                                                    const int32_t* __restrict__ ghist,
                                                                    int32_t* __restrict__ gcursor,
                                                                    int32_t* __restrict__ order)
{
    __shared__ int hist[kSizeBins];     // this workgroup's molecules per class, then its cursor inside the range
    __shared__ int start[kSizeBins];    // first position of the class in the order, then of this workgroup's range
    const int tid = threadIdx.x;
    if (tid < kSizeBins) hist[tid] = 0;
    __syncthreads();
    const int m = blockIdx.x * kOrderThreads + tid;
    int bin = 0;
    if (m < n_mols) {
        bin = size_bin(MACs[m]);
        atomicAdd(&hist[bin], 1);
    }
    __shared__ int total[kSizeBins];    // molecules per class in the whole batch
    if (tid < kSizeBins) total[tid] = ghist[tid];
    __syncthreads();
    if (tid < kSizeBins) {
        int run = 0;                    // exclusive prefix: every thread adds up the classes before its own
        for (int b = 0; b < tid; ++b) run += total[b];
        start[tid] = run;
    }
    __syncthreads();
    if (tid < kSizeBins) {
        const int mine = hist[tid];
        if (mine > 0) start[tid] += atomicAdd(&gcursor[tid], mine);
        hist[tid] = 0;
    }
    __syncthreads();
    if (m < n_mols) order[start[bin] + atomicAdd(&hist[bin], 1)] = m;
    // the four totals that tell a host which kernels have work (behind the cursors)
    if (blockIdx.x == 0 && tid < kSizeClasses) {
        const int lo = tid == 0 ? 0 : tid == 1 ? 33 : tid == 2 ? 65 : 257;          // atom counts of the class
        const int hi = tid == 0 ? 32 : tid == 1 ? 64 : tid == 2 ? 256 : 257;
        int sum = 0;
        for (int b = size_bin(hi); b <= size_bin(lo); ++b) sum += total[b];
        gcursor[kSizeBins + tid] = sum;
    }
}
}  // namespace

// `order` holds n_mols + kSizeOrderScratch entries of device memory owned by the caller: the indices, the class
// counts, the cursors.
hipError_t launch_size_order(const int32_t* MACs, int32_t n_mols, int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    int32_t* scratch = order + n_mols;
    size_clear_kernel<<<dim3(1), dim3(kSizeOrderScratch), 0, stream>>>(scratch);
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kOrderThreads - 1) / kOrderThreads;
    size_hist_kernel<<<dim3(blocks), dim3(kOrderThreads), 0, stream>>>(MACs, n_mols, scratch);
    size_place_kernel<<<dim3(blocks), dim3(kOrderThreads), 0, stream>>>(MACs, n_mols, scratch, scratch + kSizeBins, order);
    return hipGetLastError();
}

}  // namespace khan
