// Molecules of more than 256 atoms: the sorted copy of their atoms that the workgroup-per-molecule kernels read in
// place of their LDS arrays, and the kernel that writes it.
//
// Up to 256 atoms a workgroup sorts its molecule into LDS itself.  Above that the sorted atoms live in device
// memory (a molecule of a few thousand atoms stays in L2), written once per call by large_sort_kernel, and several
// workgroups share a molecule's centres.  The atoms are sorted along a space-filling curve (by type inside a cell),
// and every 64 consecutive ones have a box around them: a centre scans only the chunks whose box reaches into its
// cutoff, and puts the partners it finds in order of type afterwards.  The partner lists, the segment tables and the
// angular phases are those of the smaller molecules; only where an atom is read from differs.
#pragma once
#include "aev_small_common.h"
#include "khan_params.h"

namespace khan {

template <typename T>
struct SortedAtoms {
    typename Fast<T>::vec4* atom;   // x, y, z, type of the atom at MOs[mol] + sorted position
    typename Fast<T>::vec4* vel;    // its incoming vector (Jacobian-vector product only), else null
    int2* aux;                      // its index inside the molecule, and its scatter index (row inside its type's bucket)
    float4* box;                    // per chunk of 64 sorted atoms: lowest x, y, z and highest x, y, z (two entries)
};

// The atoms are ordered along a space-filling curve (up to 16 x 16 x 16 cells over the molecule's extent, Morton order;
// by type inside a cell), so that 64 consecutive atoms sit close together and a centre can skip the chunks whose box lies beyond its
// cutoff.  The boxes of molecule `mol` (atoms from offset `off`) start at entry 2 * chunk_base(off, mol): molecule m has
// at most macs[m] / 64 + 1 chunks, so these ranges are disjoint as long as the offsets increase with the molecule index
// and the molecules do not overlap (the exclusive prefix sum of the atom counts; stated as a precondition in khan_aev.h).
__host__ __device__ __forceinline__ size_t chunk_base(int off, int mol) { return static_cast<size_t>(off >> 6) + static_cast<size_t>(mol); }
constexpr int kSortCellsPerDim = 16;
constexpr int kSortCells = kSortCellsPerDim * kSortCellsPerDim * kSortCellsPerDim;

__host__ __device__ __forceinline__ size_t round_up_256(size_t v) { return (v + 255u) & ~static_cast<size_t>(255u); }

template <typename T>
__host__ inline size_t sorted_atoms_bytes(int64_t n_atoms, int32_t n_mols, bool with_vel)
{
    const size_t vec = round_up_256(sizeof(typename Fast<T>::vec4) * static_cast<size_t>(n_atoms));
    return vec * (with_vel ? 2 : 1) + round_up_256(sizeof(int2) * static_cast<size_t>(n_atoms)) +
           round_up_256(2 * sizeof(float4) * (static_cast<size_t>(n_atoms) / 64 + static_cast<size_t>(n_mols) + 1));
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
    s.box = reinterpret_cast<float4*>(p);
    return s;
}

// Does chunk `ch` (of n_chunks; boxes[2 ch], boxes[2 ch + 1] = its lowest and highest coordinates) come within the
// radial cutoff of the point (cx, cy, cz)?  The boxes are in float whatever the precision of the coordinates: the
// margin covers their rounding.
__device__ __forceinline__ bool chunk_in_reach(const float4* boxes, int ch, int n_chunks, float cx, float cy, float cz)
{
    if (ch >= n_chunks) return false;
    const float4 lo = boxes[2 * ch], hi = boxes[2 * ch + 1];
    const float dx = fmaxf(fmaxf(lo.x - cx, cx - hi.x), 0.0f);
    const float dy = fmaxf(fmaxf(lo.y - cy, cy - hi.y), 0.0f);
    const float dz = fmaxf(fmaxf(lo.z - cz, cz - hi.z), 0.0f);
    constexpr float reach = kR_Rc_f + 0.01f;
    return dx * dx + dy * dy + dz * dz < reach * reach;
}

// Fills `sorted` for every molecule of more than 256 atoms (stable counting sort by type and cell, one workgroup per
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
