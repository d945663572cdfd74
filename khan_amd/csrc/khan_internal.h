// Internal (C++) launch interface between the C-ABI layer and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace khan {

// Pointers to the four per-type buckets (H, C, N, O), passed to kernels by value.
template <typename T>
struct Buckets {
    T* p[4];
};

// ---- general-shape AEV kernels (any molecule size, any neighbour count) ----
template <typename T>
hipError_t launch_fwd_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, Buckets<T> out, int min_atoms, const int32_t* order,
                              hipStream_t stream);

// Jacobian applied to per-atom vectors (VX, VY, VZ): one 384-wide row per atom, laid out like the forward's
template <typename T>
hipError_t launch_jvp_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, const T* VX, const T* VY, const T* VZ, Buckets<T> out,
                              int min_atoms, const int32_t* order, hipStream_t stream);

// ---- AEV forward for molecules of up to 64 atoms (larger molecules are skipped) ----
constexpr int kSmallMaxAtoms = 64;      // what one wavefront can hold
// where a medium-molecule kernel exists, molecules above this size go to it: one wavefront working through a
// dense 64-atom molecule alone takes as long as the rest of a batch
constexpr int kSmallPreferredMax = 32;
template <typename T>
hipError_t launch_fwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<T> out,
                            int max_atoms, const int32_t* order, hipStream_t stream);

template <typename T>
hipError_t launch_jvp_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, const T* VX,
                            const T* VY, const T* VZ, Buckets<T> out, const int32_t* order, hipStream_t stream);

// ---- AEV forward for molecules of min_atoms to 256 atoms, one workgroup per molecule (other sizes are skipped) ----
constexpr int kMediumMaxAtoms = 256;
template <typename T>
hipError_t launch_fwd_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, Buckets<T> out, int min_atoms, const int32_t* order, hipStream_t stream);
// the same kernel as Jacobian-vector product
template <typename T>
hipError_t launch_jvp_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, const T* VX, const T* VY, const T* VZ,
                             Buckets<T> out, int min_atoms, const int32_t* order, hipStream_t stream);

// ---- molecules of more than 256 atoms: the same kernels reading a type-sorted copy of the atoms from `scratch`
// (large_scratch_bytes bytes of device memory, 256-byte aligned; with_vectors for the Jacobian-vector product) ----
template <typename T>
size_t large_scratch_bytes(int64_t n_atoms, int32_t n_mols, bool with_vectors);
// forward, or with VX/VY/VZ the Jacobian-vector product
template <typename T>
hipError_t launch_fwd_large(const T* X, const T* Y, const T* Z, const int32_t* A,
                            const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                            const int32_t* SIs, const T* VX, const T* VY, const T* VZ, Buckets<T> out,
                            const int32_t* order, void* scratch, int64_t n_atoms, hipStream_t stream);

// backward (the molecules' gradients need no zeroing beforehand)
template <typename T>
hipError_t launch_bwd_large(const T* X, const T* Y, const T* Z, const int32_t* A,
                            const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                            const int32_t* SIs, Buckets<const T> g, T* gX, T* gY, T* gZ,
                            const int32_t* order, void* scratch, int64_t n_atoms, hipStream_t stream);

template <typename T>
hipError_t launch_bwd_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, Buckets<const T> g, T* gX, T* gY,
                             T* gZ, int min_atoms, const int32_t* order, bool walk_in_order, bool reproducible,
                             hipStream_t stream);

template <typename T>
hipError_t launch_bwd_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, Buckets<const T> g, T* gX, T* gY, T* gZ,
                              int64_t n_atoms, int min_atoms, const int32_t* order, hipStream_t stream);
template <typename T>
hipError_t launch_bwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<const T> g,
                            T* gX, T* gY, T* gZ, int max_atoms, const int32_t* order, hipStream_t stream);

// ---- integer path ----
hipError_t launch_mol_offsets(const int32_t* mol_idxs, int64_t n_atoms, int32_t n_mols,
                              int32_t* MACs, int32_t* MOs, hipStream_t stream);
hipError_t launch_ani_sort(const int32_t* A, int64_t n_atoms, int32_t* scatter, int32_t* gather,
                           int32_t* counts4, hipStream_t stream);

// Molecule indices by decreasing atom count.  `order` holds n_mols + kSizeOrderScratch ints: the indices, then the
// number of molecules per size (kSizeBins entries, bin = size_bin(atom count)), then the pass's cursors, then the
// number of molecules of up to 32 atoms, of 33..64, of 65..256 and of more (kSizeClasses entries: what a host needs
// to know which kernels have work).
// Every `order` argument of the launchers above is such an array (or null): the kernels for larger molecules read
// the class counts behind the indices to leave at once when the batch holds no molecule for them.
// Kernels only (the counts are cleared by a small kernel), so the sequence can be recorded into a graph.
constexpr int kSizeBins = 258;    // atom counts 0..256 and "more", largest first
constexpr int kSizeClasses = 4;
constexpr int kSizeOrderScratch = 2 * kSizeBins + kSizeClasses;
__host__ __device__ __forceinline__ int size_bin(int n)
{
    const int c = n < 0 ? 0 : n > kSizeBins - 1 ? kSizeBins - 1 : n;
    return kSizeBins - 1 - c;
}
hipError_t launch_size_order(const int32_t* MACs, int32_t n_mols, int32_t* order, hipStream_t stream);

// zeros to an array of n elements (outputs that no molecule covers)
template <typename T>
hipError_t launch_zero(T* a, int64_t n, hipStream_t stream);

// per-molecule sums of the four per-type output vectors (atom g's value is bucket[as[g]][sis[g]]), and the way back
template <typename T>
hipError_t launch_mol_sum(Buckets<const T> in, const int32_t* A, const int32_t* SIs, const int32_t* MOs, const int32_t* MACs,
                          int32_t n_mols, T* e, hipStream_t stream);
template <typename T>
hipError_t launch_mol_sum_grad(const T* e_grad, const int32_t* A, const int32_t* SIs, const int32_t* MOs, const int32_t* MACs,
                               int32_t n_mols, Buckets<T> out, hipStream_t stream);

// ---- first dense layer behind the featurizer: out_t = act(rows_t . W_t + b_t) for the four types, float32 ----
// rows[t]: [n[t], 384]; wt[t]: [128, 384] (the weights transposed); bias[t]: [128]; out[t]: [n[t], 128]
hipError_t launch_dense(const float* const rows[4], const int32_t n[4], int32_t k, int32_t n_out,
                        const float* const wt[4], const float* const bias[4], bool celu, float alpha,
                        const float* const deriv_of[4], float* const out[4], hipStream_t stream);
// the last hidden layer (n_out = 64) with the output layer folded into its epilogue: head_out[t][r] = out[t][r, :] . head_w[t] + head_b[t][0]
hipError_t launch_dense_head(const float* const rows[4], const int32_t n[4], int32_t k, int32_t n_out,
                             const float* const wt[4], const float* const bias[4], bool celu, float alpha,
                             const float* const head_w[4], const float* const head_b[4], float* const out[4],
                             float* const head_out[4], hipStream_t stream);
// and the way back: rows built from scale[t][r] * head_w[t][c] * CELU'(deriv_of[t][r, c])
hipError_t launch_dense_head_grad(const float* const scale[4], const float* const head_w[4], const int32_t n[4], int32_t k,
                                  int32_t n_out, const float* const wt[4], float alpha, const float* const deriv_of[4],
                                  float* const out[4], hipStream_t stream);
// the whole 384-128-128-64-1 CELU network of the four types in one launch, forward and (grad non-null) back to the rows
hipError_t launch_networks_fused(const float* const rows[4], const int32_t n[4],
                                 const float* const w1t[4], const float* const w2t[4], const float* const w3t[4],
                                 const float* const w1[4], const float* const w2[4], const float* const w3[4],
                                 const float* const b1[4], const float* const b2[4], const float* const b3[4],
                                 const float* const w4[4], const float* const b4[4], const float* const scale[4],
                                 float alpha, float* const value[4], float* const grad[4], const void* packed,
                                 hipStream_t stream);
size_t networks_packed_bytes();
hipError_t launch_networks_pack(const float* const w1t[4], const float* const w2t[4], const float* const w3t[4],
                                const float* const w1[4], const float* const w2[4], const float* const w3[4],
                                void* packed, hipStream_t stream);
hipError_t launch_dense_first(const float* const rows[4], const int32_t n[4], const float* const wt[4],
                              const float* const bias[4], bool celu, float alpha, float* const out[4],
                              hipStream_t stream);

// ---- charges: pair energy K q_i q_j (1 - f_C(r)) / r; damped = false drops f_C (plain Coulomb) ----
template <typename T>
hipError_t launch_charge_energy(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                                const int32_t* MACs, int32_t n_mols, bool damped, T K, T* E, hipStream_t stream);
template <typename T>
hipError_t launch_charge_grad(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                              const int32_t* MACs, int32_t n_mols, const T* grads, bool damped, T K, T* q_grads,
                              T* gX, T* gY, T* gZ, T* E, hipStream_t stream);     // E (may be null): the energies as well

// ---- wavefront helpers (64 lanes) ----
__device__ __forceinline__ unsigned long long wave_ballot(bool p) { return __ballot(p); }
__device__ __forceinline__ int lowest_bit(unsigned long long m) { return __ffsll(m) - 1; }
template <typename T>
__device__ __forceinline__ T wave_get(T v, int src) { return __shfl(v, src, 64); }
template <typename T>
__device__ __forceinline__ T half_sum(T v)   // sum over the 32 lanes of this half-wave
{
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    v += __shfl_xor(v, 8, 64);
    v += __shfl_xor(v, 16, 64);
    return v;
}
template <typename T>
__device__ __forceinline__ T wave_sum(T v) { v = half_sum(v); return v + __shfl_xor(v, 32, 64); }
// orders this wave's LDS traffic: earlier LDS writes by any lane are visible to later LDS reads
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Calls body(mol) for every molecule whose atom count lies in [lo, hi].  The workgroup walks the molecules
// with the grid's stride; each thread looks at one molecule's count, the wavefronts publish ballots, and
// all threads then visit the selected molecules together (body may use __syncthreads).  A launch in
// which (nearly) every molecule belongs to another kernel therefore costs one load per thread, not a
// dependent load per molecule.  `want` is shared memory, one word per wavefront of the workgroup.  With
// `order` (molecule indices by decreasing size) the molecules are visited in that order; with `size_counts`
// (molecules per size class) a workgroup first checks that the batch holds a molecule in range.
template <typename Body>
__device__ __forceinline__ void for_each_molecule_in_range(const int32_t* __restrict__ MACs, int32_t n_mols,
                                                           int lo, int hi, unsigned long long* want,
                                                           const int32_t* __restrict__ order,
                                                           const int32_t* __restrict__ size_counts, Body body)
{
    const int tid = threadIdx.x, nthreads = blockDim.x, nwaves = nthreads >> 6;
    if (size_counts) {          // molecules per size class: is there anything in [lo, hi] at all?
        int any = 0;
        for (int b = size_bin(hi) + tid; b <= size_bin(lo); b += nthreads) any |= size_counts[b];
        if (!__syncthreads_or(any)) return;
    }
    for (long long base = blockIdx.x; base < n_mols; base += static_cast<long long>(gridDim.x) * nthreads) {
        const long long m = base + static_cast<long long>(tid) * gridDim.x;
        bool wanted = false;
        int mol = 0;                          // position m of the size order, when one is given
        if (m < n_mols) {
            mol = order ? order[m] : static_cast<int>(m);
            const int n = MACs[mol];
            wanted = n >= lo && n <= hi;
        }
        const unsigned long long mask = __ballot(wanted);
        __syncthreads();                      // everyone is done reading the previous round's words
        if ((tid & 63) == 0) want[tid >> 6] = mask;
        __syncthreads();
        for (int w = 0; w < nwaves; ++w) {
            const unsigned long long word = want[w];
            unsigned lo32 = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(word)));
            unsigned hi32 = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(word >> 32)));
            unsigned long long mm = (static_cast<unsigned long long>(hi32) << 32) | lo32;
            while (mm) {
                const int b = __ffsll(static_cast<long long>(mm)) - 1;
                mm &= mm - 1;
                const long long pos = base + static_cast<long long>(w * 64 + b) * gridDim.x;
                body(order ? __builtin_amdgcn_readfirstlane(order[pos]) : static_cast<int>(pos));
            }
        }
    }
}

}  // namespace khan
