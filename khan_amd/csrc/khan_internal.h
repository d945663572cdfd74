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
                              const int32_t* SIs, Buckets<T> out, int min_atoms, hipStream_t stream);

// Jacobian applied to per-atom vectors (VX, VY, VZ): one 384-wide row per atom, laid out like the forward's
template <typename T>
hipError_t launch_jvp_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, const T* VX, const T* VY, const T* VZ, Buckets<T> out,
                              int min_atoms, hipStream_t stream);

// ---- AEV forward for molecules of up to 64 atoms (larger molecules are skipped) ----
constexpr int kSmallMaxAtoms = 64;
template <typename T>
hipError_t launch_fwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<T> out,
                            hipStream_t stream);

template <typename T>
hipError_t launch_jvp_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, const T* VX,
                            const T* VY, const T* VZ, Buckets<T> out, hipStream_t stream);

// ---- AEV forward for molecules of 65 to 256 atoms, float32 (other sizes are skipped) ----
constexpr int kMediumMaxAtoms = 256;
hipError_t launch_fwd_medium_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                 const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                 const int32_t* SIs, Buckets<float> out, hipStream_t stream);

hipError_t launch_bwd_medium_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                 const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                 const int32_t* SIs, Buckets<const float> g, float* gX, float* gY,
                                 float* gZ, hipStream_t stream);

template <typename T>
hipError_t launch_bwd_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, Buckets<const T> g, T* gX, T* gY, T* gZ,
                              int64_t n_atoms, int min_atoms, hipStream_t stream);
template <typename T>
hipError_t launch_bwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<const T> g,
                            T* gX, T* gY, T* gZ, hipStream_t stream);

// ---- integer path ----
hipError_t launch_mol_offsets(const int32_t* mol_idxs, int64_t n_atoms, int32_t n_mols,
                              int32_t* MACs, int32_t* MOs, hipStream_t stream);
hipError_t launch_ani_sort(const int32_t* A, int64_t n_atoms, int32_t* scatter, int32_t* gather,
                           int32_t* counts4, hipStream_t stream);

// ---- charges ----
template <typename T>
hipError_t launch_charge_energy(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                                const int32_t* MACs, int32_t n_mols, T* E, hipStream_t stream);
template <typename T>
hipError_t launch_charge_grad(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                              const int32_t* MACs, int32_t n_mols, const T* grads, T* q_grads,
                              T* gX, T* gY, T* gZ, hipStream_t stream);

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

}  // namespace khan
