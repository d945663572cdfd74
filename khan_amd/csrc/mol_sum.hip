// Per-molecule sums of the atomic networks' outputs, and the way back.
//
// The reference gathers the four per-type output vectors to the batch's atom order and sums them by molecule
// (khan/model/nn.py:165-177: tf.gather(tf.concat(...), gather_idxs), then tf.segment_sum by molecule index).  Here a
// molecule's atoms find their values directly in the four buckets (type as[g], row sis[g]) and sixteen lanes add them
// up in a fixed order: one launch, no gathered copy, and the same bits on every run.  On the way back every atom's
// bucket entry receives its molecule's gradient.
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

namespace {

constexpr int kLanesPerMol = 16;
constexpr int kMolsPerBlock = 256 / kLanesPerMol;

template <typename T>
__global__ __launch_bounds__(256) void mol_sum_kernel(Buckets<const T> in, const int32_t* __restrict__ A,
                                                      const int32_t* __restrict__ SIs, const int32_t* __restrict__ MOs,
                                                      const int32_t* __restrict__ MACs, int32_t n_mols, T* __restrict__ e)
{
    const int sub = threadIdx.x & (kLanesPerMol - 1);
    const int mol = static_cast<int>(blockIdx.x) * kMolsPerBlock + static_cast<int>(threadIdx.x / kLanesPerMol);
    T acc = T(0);
    if (mol < n_mols) {
        const int off = MOs[mol], n = MACs[mol];
        for (int i = sub; i < n; i += kLanesPerMol) {
            const int g = off + i;
            const int t = fold_type(A[g]);
            const T* bucket = t == 0 ? in.p[0] : t == 1 ? in.p[1] : t == 2 ? in.p[2] : in.p[3];
            acc += bucket[SIs[g]];
        }
    }
    // the sixteen partial sums of a molecule, always added in the same order
#pragma unroll
    for (int d = kLanesPerMol / 2; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
    if (sub == 0 && mol < n_mols) e[mol] = acc;
}

template <typename T>
__global__ __launch_bounds__(256) void mol_sum_grad_kernel(const T* __restrict__ e_grad, const int32_t* __restrict__ A,
                                                           const int32_t* __restrict__ SIs, const int32_t* __restrict__ MOs,
                                                           const int32_t* __restrict__ MACs, int32_t n_mols, Buckets<T> out)
{
    const int sub = threadIdx.x & (kLanesPerMol - 1);
    const int mol = static_cast<int>(blockIdx.x) * kMolsPerBlock + static_cast<int>(threadIdx.x / kLanesPerMol);
    if (mol >= n_mols) return;
    const int off = MOs[mol], n = MACs[mol];
    const T g_m = e_grad[mol];
    for (int i = sub; i < n; i += kLanesPerMol) {
        const int g = off + i;
        const int t = fold_type(A[g]);
        T* bucket = t == 0 ? out.p[0] : t == 1 ? out.p[1] : t == 2 ? out.p[2] : out.p[3];
        bucket[SIs[g]] = g_m;
    }
}

}  // namespace

template <typename T>
hipError_t launch_mol_sum(Buckets<const T> in, const int32_t* A, const int32_t* SIs, const int32_t* MOs, const int32_t* MACs,
                          int32_t n_mols, T* e, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kMolsPerBlock - 1u) / kMolsPerBlock;
    mol_sum_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(in, A, SIs, MOs, MACs, n_mols, e);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_mol_sum_grad(const T* e_grad, const int32_t* A, const int32_t* SIs, const int32_t* MOs, const int32_t* MACs,
                               int32_t n_mols, Buckets<T> out, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kMolsPerBlock - 1u) / kMolsPerBlock;
    mol_sum_grad_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(e_grad, A, SIs, MOs, MACs, n_mols, out);
    return hipGetLastError();
}

template hipError_t launch_mol_sum<float>(Buckets<const float>, const int32_t*, const int32_t*, const int32_t*, const int32_t*, int32_t, float*, hipStream_t);
template hipError_t launch_mol_sum<double>(Buckets<const double>, const int32_t*, const int32_t*, const int32_t*, const int32_t*, int32_t, double*, hipStream_t);
template hipError_t launch_mol_sum_grad<float>(const float*, const int32_t*, const int32_t*, const int32_t*, const int32_t*, int32_t, Buckets<float>, hipStream_t);
template hipError_t launch_mol_sum_grad<double>(const double*, const int32_t*, const int32_t*, const int32_t*, const int32_t*, int32_t, Buckets<double>, hipStream_t);

}  // namespace khan
