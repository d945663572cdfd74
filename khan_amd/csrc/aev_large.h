// Molecules of more than 256 atoms: the type-sorted copy of their atoms that the workgroup-per-molecule kernels
// read in place of their LDS arrays, and the kernel that writes it.
//
// Up to 256 atoms a workgroup sorts its molecule into LDS itself.  Above that the sorted atoms live in device
// memory (a molecule of a few thousand atoms stays in L2), written once per call by large_sort_kernel, and several
// workgroups share a molecule's centres.  The partner lists, the segment tables and the angular phases are those
// of the smaller molecules; only where an atom is read from differs.
#pragma once
#include "aev_small_common.h"

namespace khan {

template <typename T>
struct SortedAtoms {
    typename Fast<T>::vec4* atom;   // x, y, z, type of the atom at MOs[mol] + sorted position
    typename Fast<T>::vec4* vel;    // its incoming vector (Jacobian-vector product only), else null
    int2* aux;                      // its index inside the molecule, and its scatter index (row inside its type's bucket)
    int4* tbase;                    // per molecule: sorted position of the first atom of each type
};

__host__ __device__ __forceinline__ size_t round_up_256(size_t v) { return (v + 255u) & ~static_cast<size_t>(255u); }

template <typename T>
__host__ inline size_t sorted_atoms_bytes(int64_t n_atoms, int32_t n_mols, bool with_vel)
{
    const size_t vec = round_up_256(sizeof(typename Fast<T>::vec4) * static_cast<size_t>(n_atoms));
    return vec * (with_vel ? 2 : 1) + round_up_256(sizeof(int2) * static_cast<size_t>(n_atoms)) +
           round_up_256(sizeof(int4) * static_cast<size_t>(n_mols));
}

// the arrays inside one allocation of sorted_atoms_bytes (256-byte aligned)
template <typename T>
__host__ inline SortedAtoms<T> carve_sorted_atoms(void* scratch, int64_t n_atoms, int32_t n_mols, bool with_vel)
{
    typedef typename Fast<T>::vec4 vec4;
    char* p = static_cast<char*>(scratch);
    const size_t vec = round_up_256(sizeof(vec4) * static_cast<size_t>(n_atoms));
    SortedAtoms<T> s;
    s.atom = reinterpret_cast<vec4*>(p);
    p += vec;
    s.vel = nullptr;
    if (with_vel) {
        s.vel = reinterpret_cast<vec4*>(p);
        p += vec;
    }
    s.aux = reinterpret_cast<int2*>(p);
    p += round_up_256(sizeof(int2) * static_cast<size_t>(n_atoms));
    s.tbase = reinterpret_cast<int4*>(p);
    return s;
}

// Fills `sorted` for every molecule of more than 256 atoms (stable counting sort by type, one workgroup per
// molecule); with gX the molecule's gradients are zeroed as well (the backward kernel then only adds).
template <typename T>
hipError_t launch_large_sort(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                             const int32_t* MACs, int32_t n_mols, const int32_t* SIs, const T* VX, const T* VY,
                             const T* VZ, T* gX, T* gY, T* gZ, const int32_t* order, SortedAtoms<T> sorted,
                             hipStream_t stream);

// Grid of the kernels for large molecules: x = molecules in flight (at most 32), y = workgroups that share a
// molecule's centres (64; more when the batch has few molecules, so that one large molecule alone still fills the GPU).
__host__ inline dim3 large_grid(int32_t n_mols)
{
    const unsigned columns = static_cast<unsigned>(n_mols < 32 ? n_mols : 32);
    const unsigned parts = columns >= 32 ? 64u : (2048u / columns > 1024u ? 1024u : 2048u / columns);
    return dim3(columns, parts);
}

}  // namespace khan
