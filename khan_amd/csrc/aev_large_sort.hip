// Type-sorted copies of the molecules of more than 256 atoms, for the workgroup-per-molecule AEV kernels
// (aev_large.h).  One workgroup per molecule: a stable counting sort by atom type, 256 atoms per step.
#include "aev_large.h"
#include "khan_params.h"

namespace khan {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void large_sort_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    const T* __restrict__ VX, const T* __restrict__ VY, const T* __restrict__ VZ,
    T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ, const int32_t* __restrict__ order,
    SortedAtoms<T> sorted)
{
    __shared__ int wcount[4][4];               // atoms of each type held by each wavefront in the current step
    __shared__ unsigned long long want[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    for_each_molecule_in_range(MACs, n_mols, kMediumMaxAtoms + 1, INT32_MAX, want, order, order ? order + n_mols : nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);

        // ---- atoms of each type
        int tot[4] = {0, 0, 0, 0};
        for (int base = 0; base < n; base += 256) {
            const int j = base + tid;
            const int type = j < n ? fold_type(A[off + j]) : -1;
#pragma unroll
            for (int a = 0; a < 4; ++a) tot[a] += popc64(wave_ballot(type == a));
        }
        if (lane < 4) wcount[wave][lane] = sel4(lane, tot[0], tot[1], tot[2], tot[3]);
        __syncthreads();
        int run[4];                             // next free sorted position of each type (the same in every thread)
        {
            int r = 0;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                run[a] = r;
                r += wcount[0][a] + wcount[1][a] + wcount[2][a] + wcount[3][a];
            }
        }
        if (tid == 0) sorted.tbase[mol] = make_int4(run[0], run[1], run[2], run[3]);
        __syncthreads();                        // the counts are reused below

        // ---- place the atoms, 256 per step, keeping their order inside a type
        for (int base = 0; base < n; base += 256) {
            const int j = base + tid;
            const bool have = j < n;
            T x = T(0), y = T(0), z = T(0);
            int type = -1, si = 0;
            if (have) {
                x = X[off + j];
                y = Y[off + j];
                z = Z[off + j];
                type = fold_type(A[off + j]);
                si = SIs[off + j];
            }
            unsigned long long tmask[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) tmask[a] = wave_ballot(type == a);
            if (lane < 4) wcount[wave][lane] = popc64(lane == 0 ? tmask[0] : lane == 1 ? tmask[1] : lane == 2 ? tmask[2] : tmask[3]);
            __syncthreads();
            if (have) {
                int before = 0;                 // atoms of my type held by earlier wavefronts in this step
                for (int w = 0; w < wave; ++w) before += wcount[w][type];
                const unsigned long long mine = type == 0 ? tmask[0] : type == 1 ? tmask[1] : type == 2 ? tmask[2] : tmask[3];
                const int dest = off + sel4(type, run[0], run[1], run[2], run[3]) + before + popc64(mine & lt_mask);
                sorted.atom[dest] = Fast<T>::make4(x, y, z, static_cast<T>(type));
                sorted.aux[dest] = make_int2(j, si);
                if (sorted.vel) sorted.vel[dest] = Fast<T>::make4(VX[off + j], VY[off + j], VZ[off + j], T(0));
                if (gX) {
                    gX[off + j] = T(0);
                    gY[off + j] = T(0);
                    gZ[off + j] = T(0);
                }
            }
#pragma unroll
            for (int a = 0; a < 4; ++a) run[a] += wcount[0][a] + wcount[1][a] + wcount[2][a] + wcount[3][a];
            __syncthreads();                    // the next step (or molecule) overwrites the counts
        }
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
