// Sorted copies of the molecules of more than 256 atoms, for the workgroup-per-molecule AEV kernels (aev_large.h).
// One workgroup per molecule: a counting sort by (cell along a space-filling curve, atom type) that keeps the atoms'
// order inside a bin, 256 atoms per step, and the box around every 64 consecutive sorted atoms.
#include "aev_large.h"
#include "khan_params.h"

namespace khan {

namespace {

__device__ __forceinline__ int spread4(int v) { return (v & 1) | ((v & 2) << 2) | ((v & 4) << 4) | ((v & 8) << 6); }

// minimum / maximum over the wavefront
__device__ __forceinline__ float wave_min(float v)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v = fminf(v, __shfl_xor(v, d, 64));
    return v;
}
__device__ __forceinline__ float wave_maxf(float v)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
    return v;
}

template <typename T>
__global__ __launch_bounds__(256) void large_sort_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    const T* __restrict__ VX, const T* __restrict__ VY, const T* __restrict__ VZ,
    T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ, const int32_t* __restrict__ order,
    SortedAtoms<T> sorted)
{
    __shared__ int hist[4 * kSortCells];       // atoms per (cell, type); after the scan each one's next free sorted position
    __shared__ int in_step[4 * kSortCells];    // atoms per (cell, type) among the 256 of the current step (zero between steps)
    __shared__ __align__(16) int2 shared_bin[256];           // (key, thread) of the step's atoms that share their bin with another
    __shared__ int wshared[4];                 // how many of them each wavefront holds
    __shared__ __align__(16) int step_key[256];              // keys of the 256 atoms of the current step
    __shared__ float ext[4][6];                // each wavefront's share of the molecule's extent
    __shared__ int wsum[4];
    __shared__ unsigned long long want[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    for_each_molecule_in_range(MACs, n_mols, kMediumMaxAtoms + 1, INT32_MAX, want, order, order ? order + n_mols : nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);

        // ---- the molecule's extent, and the cell grid over it
        float lo[3] = {3.0e38f, 3.0e38f, 3.0e38f}, hi[3] = {-3.0e38f, -3.0e38f, -3.0e38f};
        // (one workgroup walks the whole molecule: eight atoms' loads in flight per thread in this and the next loop)
#pragma unroll 8
        for (int j = tid; j < n; j += 256) {
            const float p[3] = {static_cast<float>(X[off + j]), static_cast<float>(Y[off + j]), static_cast<float>(Z[off + j])};
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                lo[k] = fminf(lo[k], p[k]);
                hi[k] = fmaxf(hi[k], p[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            lo[k] = wave_min(lo[k]);
            hi[k] = wave_maxf(hi[k]);
        }
        if (lane == 0) {
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                ext[wave][k] = lo[k];
                ext[wave][3 + k] = hi[k];
            }
        }
        __syncthreads();
        // cells per dimension: 4, 8 or 16 by the molecule's size (a chunk of 64 atoms spans several cells either way,
        // and the bins' bookkeeping below grows with the cube of it)
        const int g = n <= 1024 ? 4 : n <= 8192 ? 8 : kSortCellsPerDim;
        const int cells = g * g * g, bins = 4 * cells, per_thread = bins / 256;
        float scale[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            lo[k] = fminf(fminf(ext[0][k], ext[1][k]), fminf(ext[2][k], ext[3][k]));
            hi[k] = fmaxf(fmaxf(ext[0][3 + k], ext[1][3 + k]), fmaxf(ext[2][3 + k], ext[3][3 + k]));
            scale[k] = static_cast<float>(g) / fmaxf(hi[k] - lo[k], 1.0e-3f);
        }
        // (cell, type) of atom j: the cell's index along the space-filling curve, then the type
        auto key_of = [&](int j) -> int {
            const float p[3] = {static_cast<float>(X[off + j]), static_cast<float>(Y[off + j]), static_cast<float>(Z[off + j])};
            int c[3];
#pragma unroll
            for (int k = 0; k < 3; ++k) c[k] = min(max(static_cast<int>((p[k] - lo[k]) * scale[k]), 0), g - 1);
            return (spread4(c[0]) | (spread4(c[1]) << 1) | (spread4(c[2]) << 2)) * 4 + fold_type(A[off + j]);
        };

        // ---- atoms per (cell, type)
        for (int b = tid; b < bins; b += 256) {
            hist[b] = 0;
            in_step[b] = 0;
        }
        __syncthreads();
#pragma unroll 8
        for (int j = tid; j < n; j += 256) atomicAdd(&hist[key_of(j)], 1);
        __syncthreads();
        // ---- exclusive prefix sum over the bins: per_thread consecutive bins per thread
        {
            int local = 0;
            for (int q = 0; q < per_thread; ++q) local += hist[per_thread * tid + q];
            int incl = local;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int v = __shfl_up(incl, d, 64);
                if (lane >= d) incl += v;
            }
            if (lane == 63) wsum[wave] = incl;
            __syncthreads();
            int run = incl - local;
            for (int w = 0; w < wave; ++w) run += wsum[w];
            for (int q = 0; q < per_thread; ++q) {
                const int c = hist[per_thread * tid + q];
                hist[per_thread * tid + q] = run;
                run += c;
            }
        }
        __syncthreads();

        // ---- place the atoms, 256 per step, in index order inside a (cell, type): the result does not depend on timing.
        // An atom's data are fetched one step ahead, so that the loads run under the previous step's ranking.
        struct Fetched {
            T x, y, z, vx, vy, vz;
            int type, si;
        };
        auto fetch = [&](int j) -> Fetched {
            Fetched f;
            f.x = f.y = f.z = f.vx = f.vy = f.vz = T(0);
            f.type = 0;
            f.si = 0;
            if (j < n) {
                f.x = X[off + j];
                f.y = Y[off + j];
                f.z = Z[off + j];
                f.type = fold_type(A[off + j]);
                f.si = SIs[off + j];
                if (sorted.vel) {
                    f.vx = VX[off + j];
                    f.vy = VY[off + j];
                    f.vz = VZ[off + j];
                }
            }
            return f;
        };
        Fetched next = fetch(tid);
        for (int base = 0; base < n; base += 256) {
            const int j = base + tid;
            const bool have = j < n;
            const Fetched cur = next;
            next = fetch(j + 256);
            int key = -1 - tid;                                    // (no two threads without an atom match)
            if (have) {
                const float p[3] = {static_cast<float>(cur.x), static_cast<float>(cur.y), static_cast<float>(cur.z)};
                int c[3];
#pragma unroll
                for (int k = 0; k < 3; ++k) c[k] = min(max(static_cast<int>((p[k] - lo[k]) * scale[k]), 0), g - 1);
                key = (spread4(c[0]) | (spread4(c[1]) << 1) | (spread4(c[2]) << 2)) * 4 + cur.type;
            }
            // Rank among the step's atoms of the same bin, by thread.  In a large molecule most atoms are alone in their
            // bin within a step: the atoms that are not are listed (in thread order) and only they compare keys, with
            // that list.  When the list is long (small molecules, few bins) every atom compares with the 255 others.
            step_key[tid] = key;
            if (have) atomicAdd(&in_step[key], 1);
            __syncthreads();
            const bool shares = have && in_step[key] > 1;
            const unsigned long long smask = wave_ballot(shares);
            if (lane == 0) wshared[wave] = popc64(smask);
            __syncthreads();
            int before = 0, n_shared = 0;
            for (int w = 0; w < 4; ++w) {
                before += w < wave ? wshared[w] : 0;
                n_shared += wshared[w];
            }
            if (shares) shared_bin[before + popc64(smask & ((1ull << lane) - 1ull))] = make_int2(key, tid);
            __syncthreads();
            int rank = 0;
            if (n_shared > 48) {
#pragma unroll 8
                for (int t = 0; t < 256; t += 4) {
                    const int4 k4 = *reinterpret_cast<const int4*>(&step_key[t]);
                    rank += (k4.x == key && t < tid) + (k4.y == key && t + 1 < tid) + (k4.z == key && t + 2 < tid) +
                            (k4.w == key && t + 3 < tid);
                }
            } else if (shares) {
                for (int q = 0; q < n_shared; ++q) {
                    const int2 e = shared_bin[q];
                    rank += (e.x == key && e.y < tid);
                }
            }
            const int dest = have ? off + hist[key] + rank : 0;
            __syncthreads();                    // every thread has read its bin's position and the step's counts
            if (have) in_step[key] = 0;
            if (have) {
                atomicAdd(&hist[key], 1);
                sorted.atom[dest] = Fast<T>::make4(cur.x, cur.y, cur.z, static_cast<T>(cur.type));
                sorted.aux[dest] = make_int2(j, cur.si);
                if (sorted.vel) sorted.vel[dest] = Fast<T>::make4(cur.vx, cur.vy, cur.vz, T(0));
                if (gX) {
                    gX[off + j] = T(0);
                    gY[off + j] = T(0);
                    gZ[off + j] = T(0);
                }
            }
            __syncthreads();                    // the bins are up to date, the keys may be overwritten
        }

        // ---- the box around every 64 consecutive sorted atoms
        __threadfence();
        __syncthreads();                        // the workgroup's stores to sorted.atom are visible to its loads
        const size_t cb = chunk_base(off, mol);
        const int n_chunks = (n + 63) >> 6;
        for (int c = wave; c < n_chunks; c += 4) {
            const int j = 64 * c + lane;
            float p[3] = {0.0f, 0.0f, 0.0f};
            const bool have = j < n;
            if (have) {
                const typename Fast<T>::vec4 a = sorted.atom[off + j];
                p[0] = static_cast<float>(a.x);
                p[1] = static_cast<float>(a.y);
                p[2] = static_cast<float>(a.z);
            }
            float blo[3], bhi[3];
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                blo[k] = wave_min(have ? p[k] : 3.0e38f);
                bhi[k] = wave_maxf(have ? p[k] : -3.0e38f);
            }
            if (lane == 0) {
                sorted.box[2 * (cb + c)] = make_float4(blo[0], blo[1], blo[2], 0.0f);
                sorted.box[2 * (cb + c) + 1] = make_float4(bhi[0], bhi[1], bhi[2], 0.0f);
            }
        }
        __syncthreads();                        // the next molecule reuses the shared arrays
    });
}

}  // namespace

template <typename T>
hipError_t launch_large_sort(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                             const int32_t* MACs, int32_t n_mols, const int32_t* SIs, const T* VX, const T* VY,
                             const T* VZ, T* gX, T* gY, T* gZ, const int32_t* order, SortedAtoms<T> sorted,
                             hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = static_cast<unsigned>(n_mols < 1024 ? n_mols : 1024);
    large_sort_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, VX, VY, VZ, gX, gY, gZ,
                                                             order, sorted);
    return hipGetLastError();
}

template hipError_t launch_large_sort<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const float*, const float*, const float*, float*, float*, float*, const int32_t*, SortedAtoms<float>, hipStream_t);
template hipError_t launch_large_sort<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const double*, const double*, const double*, double*, double*, double*, const int32_t*, SortedAtoms<double>, hipStream_t);

}  // namespace khan
