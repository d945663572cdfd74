// Damped-Coulomb charge energy and its gradients on gfx950.
//
// Reference: gpu_featurizer/ani_charges.cpp:58-71 (energy), 138-160 (dE/dq):
//     E_m = sum_{i<j in m} K q_i q_j (1 - f_C(r_ij, R_Rc)) / r_ij,   K = 0.529176917f, R_Rc = 4.6f
//     dL/dq_i = g_m * sum_{j != i} K q_j (1 - f_C(r_ij)) / r_ij
// f_C(r) = 0.5 cos(pi r / Rc) + 0.5 for r <= Rc, else 0 (so pairs beyond Rc are plain K q q / r).
// The coordinate gradient has no reference counterpart (the reference returns None for x, y, z,
// khan/training/trainer_multi_tower.py:112-119); it is the closed form
//     dL/dx_i = g_m K q_i sum_{j != i} q_j d/dr[(1 - f_C)/r] (x_i - x_j)/r.
//
// One wavefront per molecule.  Up to 64 atoms a step evaluates 64 (i, j) pairs at once -- 4 atoms i x 16
// partners j for molecules of up to 16 atoms, 2 x 32 up to 32, 1 x 64 above -- with the partners' data
// held in the lanes, and the sums over j are in-wave DPP reductions (a lane per atom i walking all j
// would leave four fifths of the lanes idle on a 12-atom molecule).  Molecules of 65 to 256 atoms go to a
// second kernel that tiles the molecule through LDS (charge_tile_kernel below).  Above 256 atoms several
// workgroups share a molecule: all pairs, the partners tiled through LDS (charge_large_kernel).  Each output
// element is written once, no atomics and no pre-zeroing -- except the energy of a molecule of more than 256 atoms,
// which is the sum of its workgroups' shares.
#include "aev_small_common.h"

namespace khan {

namespace {

// Distance arithmetic per precision.  float: the hardware reciprocal square root with one Newton step, the hardware
// reciprocal and the minimax cutoff polynomials of the AEV kernels.  double: no library call either (sqrt_and_rcp and
// the Taylor cutoff of aev_small_common.h) -- the library's sqrt, division, cos and sin come to some 250 instructions
// per pair, most of them range reduction and special cases that cannot occur here, and made these kernels run at
// 2.6 % of the double-precision vector peak.
template <typename T> struct ChargeMath;
template <> struct ChargeMath<float> {
    // r = sqrt(d2) and 1/r (0 for d2 = 0)
    static __device__ __forceinline__ void dist(float d2, float& r, float& inv)
    {
        r = Fast<float>::sqrt_rn(d2);
        inv = d2 > 0.0f ? Fast<float>::rcp(r) : 0.0f;
    }
    // f_C(r, R_Rc) and its derivative, for r <= R_Rc
    static __device__ __forceinline__ void cutoff(float r, float& fc, float& dfc)
    {
        Fast<float>::cutoff_grad(r, kR_Rc_f, fc, dfc);
    }
};
template <> struct ChargeMath<double> {
    static __device__ __forceinline__ void dist(double d2, double& r, double& inv) { sqrt_and_rcp(d2, r, inv); }
    static __device__ __forceinline__ void cutoff(double r, double& fc, double& dfc)
    {
        Fast<double>::cutoff_grad(r, static_cast<double>(kR_Rc_f), fc, dfc);
    }
};

// kDamped = false drops the cutoff function: plain Coulomb pairs q_i q_j / r (the reference's op is the damped form)
template <typename T, bool kDamped>
__device__ __forceinline__ void pair_terms(T dx, T dy, T dz, T& u, T& dudr_over_r)
{
    T r, inv;            // coincident atoms (r = 0): inv = 0, so that (1 - f_C)/r -> 0 there and the pair pulls nowhere
    ChargeMath<T>::dist(dx * dx + dy * dy + dz * dz, r, inv);
    T fc = T(0), dfc = T(0);
    if constexpr (kDamped) {
        // evaluated in every lane and selected: a branch would be taken by nearly every wavefront anyway
        ChargeMath<T>::cutoff(r, fc, dfc);
        const bool in = r <= static_cast<T>(kR_Rc_f);
        fc = in ? fc : T(0);
        dfc = in ? dfc : T(0);
    }
    u = (T(1) - fc) * inv;                            // (1 - f_C) / r
    dudr_over_r = (-dfc * inv - u * inv) * inv;       // d/dr[(1-f_C)/r] / r
}

template <typename T, bool kDamped>
__global__ __launch_bounds__(256) void charge_energy_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const T* __restrict__ Q, const int32_t* __restrict__ MOs, const int32_t* __restrict__ MACs,
    int32_t n_mols, T K, T* __restrict__ E)
{
    const int lane = threadIdx.x & 63;
    const int64_t mol = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (mol >= n_mols) return;
    const int n = MACs[mol], off = MOs[mol];
    if (n > kSmallMaxAtoms && n <= kMediumMaxAtoms) return;      // the tile kernel's
    T acc = T(0);
    if (n <= 64) {
        const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
        const int W = 1 << logW, G = 64 >> logW;
        const int grp = lane >> logW, jl = lane & (W - 1);
        const bool jok = jl < n;
        const T xj = jok ? X[off + jl] : T(0), yj = jok ? Y[off + jl] : T(0), zj = jok ? Z[off + jl] : T(0),
                qj = jok ? Q[off + jl] : T(0);
        for (int i0 = 0; i0 < n; i0 += G) {
            const int i = i0 + grp;                      // lane i of the first group holds atom i
            const T xi = __shfl(xj, i & 63, 64), yi = __shfl(yj, i & 63, 64), zi = __shfl(zj, i & 63, 64),
                    qi = __shfl(qj, i & 63, 64);
            const bool valid = (i < n) && jok && (jl > i);
            T u, du;
            pair_terms<T, kDamped>(valid ? xi - xj : T(1), valid ? yi - yj : T(0), valid ? zi - zj : T(0), u, du);
            acc += valid ? K * qi * qj * u : T(0);
        }
        acc = wave_sum(acc);
        if (lane == 0) E[mol] = acc;
        return;
    }
    // more than 256 atoms: charge_large_kernel adds its workgroups' shares to the energy, which starts from zero here
    if (lane == 0) E[mol] = T(0);
}

template <typename T, bool kDamped>
__global__ __launch_bounds__(256) void charge_grad_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const T* __restrict__ Q, const int32_t* __restrict__ MOs, const int32_t* __restrict__ MACs,
    int32_t n_mols, const T* __restrict__ grads, T K, T* __restrict__ q_grads, T* __restrict__ gX,
    T* __restrict__ gY, T* __restrict__ gZ, T* __restrict__ E)
{
    const int lane = threadIdx.x & 63;
    const int64_t mol = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (mol >= n_mols) return;
    const int n = MACs[mol], off = MOs[mol];
    if (n > kSmallMaxAtoms && n <= kMediumMaxAtoms) return;      // the tile kernel's
    const T gK = grads[mol] * K;
    T e_acc = T(0);          // sum over atoms of q_i sum_j q_j u_ij = twice the energy / K
    if (n <= 64) {
        const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
        const int W = 1 << logW, G = 64 >> logW;
        const int grp = lane >> logW, jl = lane & (W - 1);
        const bool jok = jl < n;
        const T xj = jok ? X[off + jl] : T(0), yj = jok ? Y[off + jl] : T(0), zj = jok ? Z[off + jl] : T(0),
                qj = jok ? Q[off + jl] : T(0);
        for (int i0 = 0; i0 < n; i0 += G) {
            const int i = i0 + grp;                      // lane i of the first group holds atom i
            const T xi = __shfl(xj, i & 63, 64), yi = __shfl(yj, i & 63, 64), zi = __shfl(zj, i & 63, 64),
                    qi = __shfl(qj, i & 63, 64);
            const bool valid = (i < n) && jok && (jl != i);
            const T dx = valid ? xi - xj : T(1), dy = valid ? yi - yj : T(0), dz = valid ? zi - zj : T(0);
            T u, du;
            pair_terms<T, kDamped>(dx, dy, dz, u, du);
            const T w = valid ? qj * du : T(0);
            // sums over the W partners of the group end up in its last lane
            const T dq = group_sum_to_last_lane(valid ? qj * u : T(0), logW);
            const T fx = group_sum_to_last_lane(w * dx, logW);
            const T fy = group_sum_to_last_lane(w * dy, logW);
            const T fz = group_sum_to_last_lane(w * dz, logW);
            if (jl == W - 1 && i < n) {
                e_acc = fma(qi, dq, e_acc);
                if (q_grads) q_grads[off + i] = gK * dq;
                if (gX) {
                    gX[off + i] = gK * qi * fx;
                    gY[off + i] = gK * qi * fy;
                    gZ[off + i] = gK * qi * fz;
                }
            }
        }
        if (E) {
            e_acc = wave_sum(e_acc);
            if (lane == 0) E[mol] = T(0.5) * K * e_acc;
        }
        return;
    }
    // more than 256 atoms: charge_large_kernel's, which adds its workgroups' shares to an energy that starts from zero
    if (E && lane == 0) E[mol] = T(0);
}

// Molecules of 65 to 256 atoms: one workgroup of four wavefronts per molecule, the molecule (x, y, z, q) in LDS, one
// atom i per thread.  In round d a thread pairs its atom with atom j = (i + d) mod n, read from the tile: after
// (n-1)/2 rounds (plus half a round when n is even) every unordered pair has been evaluated exactly once -- half the
// pair evaluations of a walk over all j != i.  In a round the partners j of a wavefront's atoms are distinct, so what a
// pair contributes to its partner (dE/dq_j and the force on j) is added to the partner's slot in LDS by plain
// read-add-write, without atomics, while the atom's own side stays in registers.  Every wavefront adds into a copy of
// its own of the partner slots, so the four never wait for each other inside the rounds (a barrier per round would be
// the alternative); the copies are summed at the end.  A wavefront whose 64 atoms lie beyond the molecule sits the
// rounds out.  Every output element is written once.
template <typename T, bool kGrad> struct ChargeTile;
template <typename T> struct __align__(16) ChargeTile<T, false> {
    typename Fast<T>::vec4 in[kMediumMaxAtoms];     // x, y, z, q
    T wpart[4];
};
// (in double these are 40,960 bytes, a quarter of a compute unit's LDS to the byte: the wavefronts' partial energies
// go into the tile's first entry once the rounds are over, not into four words more that would cost the fourth workgroup)
template <typename T> struct __align__(16) ChargeTile<T, true> {
    typename Fast<T>::vec4 in[kMediumMaxAtoms];     // x, y, z, q
    typename Fast<T>::vec4 acc[4][kMediumMaxAtoms]; // partner side, per wavefront: force x, y, z and dE/dq
};

template <typename T, bool kDamped, bool kGrad>
__global__ __launch_bounds__(256) void charge_tile_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const T* __restrict__ Q, const int32_t* __restrict__ MOs, const int32_t* __restrict__ MACs,
    int32_t n_mols, const T* __restrict__ grads, T K, T* __restrict__ E, T* __restrict__ q_grads,
    T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ)
{
    typedef typename Fast<T>::vec4 vec4;
    static_assert(kMediumMaxAtoms == 256, "one atom per thread of a 256-thread workgroup");
    __shared__ ChargeTile<T, kGrad> S;
    const int i = threadIdx.x, lane = i & 63, wave = uniform(i >> 6);
    for (int mol = blockIdx.x; mol < n_mols; mol += gridDim.x) {
        const int n = uniform(MACs[mol]);
        if (n <= kSmallMaxAtoms || n > kMediumMaxAtoms) continue;
        const int off = uniform(MOs[mol]);
        const bool have = i < n;
        vec4 own = Fast<T>::make4(T(0), T(0), T(0), T(0));
        if (have) {
            own = Fast<T>::make4(X[off + i], Y[off + i], Z[off + i], Q[off + i]);
            S.in[i] = own;
        }
        if constexpr (kGrad) {
#pragma unroll
            for (int w = 0; w < 4; ++w) S.acc[w][i] = Fast<T>::make4(T(0), T(0), T(0), T(0));
        }
        __syncthreads();
        const int half = (n - 1) >> 1;
        const int rounds = (wave * 64 < n) ? half + (((n & 1) == 0) ? 1 : 0) : 0;
        T fx = T(0), fy = T(0), fz = T(0), dq = T(0), e_acc = T(0);
        for (int d = 1; d <= rounds; ++d) {
            const bool act = have && (d <= half || i < (n >> 1));     // the half round: the lower half only
            int j = i + d;
            j -= (j >= n) ? n : 0;
            const vec4 aj = S.in[act ? j : 0];
            const T dx = act ? own.x - aj.x : T(1), dy = act ? own.y - aj.y : T(0), dz = act ? own.z - aj.z : T(0);
            T u, du;
            pair_terms<T, kDamped>(dx, dy, dz, u, du);
            const T qq = act ? own.w * aj.w : T(0);
            e_acc = fma(qq, u, e_acc);
            if constexpr (kGrad) {
                if (act) {
                    dq = fma(aj.w, u, dq);
                    const T wq = qq * du;                    // q_i q_j d/dr[(1-f_C)/r] / r
                    fx = fma(wq, dx, fx);
                    fy = fma(wq, dy, fy);
                    fz = fma(wq, dz, fz);
                    vec4 pa = S.acc[wave][j];                // distinct j across the lanes of this wavefront
                    pa.x = fma(-wq, dx, pa.x);
                    pa.y = fma(-wq, dy, pa.y);
                    pa.z = fma(-wq, dz, pa.z);
                    pa.w = fma(own.w, u, pa.w);
                    S.acc[wave][j] = pa;
                }
                wave_lds_fence();                            // the next round may touch slots written here
            }
        }
        T* wpart;
        if constexpr (kGrad) {
            wpart = reinterpret_cast<T*>(&S.in[0]);
            if (E) __syncthreads();          // every wavefront has finished its rounds: the tile is free
        } else {
            wpart = S.wpart;
        }
        if (!kGrad || E) {
            e_acc = wave_sum(e_acc);
            if (lane == 0) wpart[wave] = e_acc;
        }
        __syncthreads();
        if ((!kGrad || E) && i == 0) E[mol] = K * ((wpart[0] + wpart[1]) + (wpart[2] + wpart[3]));
        if constexpr (kGrad) {
            if (have) {
                const T gK = grads[mol] * K;
                const vec4 p0 = S.acc[0][i], p1 = S.acc[1][i], p2 = S.acc[2][i], p3 = S.acc[3][i];
                if (q_grads) q_grads[off + i] = gK * (dq + ((p0.w + p1.w) + (p2.w + p3.w)));
                if (gX) {
                    // the force sums carry q_i already (wq = q_i q_j ...)
                    gX[off + i] = gK * (fx + ((p0.x + p1.x) + (p2.x + p3.x)));
                    gY[off + i] = gK * (fy + ((p0.y + p1.y) + (p2.y + p3.y)));
                    gZ[off + i] = gK * (fz + ((p0.z + p1.z) + (p2.z + p3.z)));
                }
            }
        }
        __syncthreads();         // the next molecule reuses the tile
    }
}

// Molecules of more than 256 atoms: all pairs, the partners tiled through LDS 256 at a time.  A thread owns one atom i
// of a block of 256 and sums over every partner j (each pair is evaluated from both ends: no exchange between threads, and
// every per-atom output is written once, by its owner); the workgroups of a grid column (blockIdx.y) share a molecule's
// blocks.  The energy is half the sum over atoms of q_i times the atom's sum, added to E[mol] (zeroed by
// charge_energy_kernel or charge_grad_kernel, which runs before on the same stream) by one floating-point atomic per workgroup and block: its
// last bits depend on the order of those additions.
template <typename T, bool kDamped, bool kGrad>
__global__ __launch_bounds__(256) void charge_large_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const T* __restrict__ Q, const int32_t* __restrict__ MOs, const int32_t* __restrict__ MACs,
    int32_t n_mols, const T* __restrict__ grads, T K, T* __restrict__ E, T* __restrict__ q_grads,
    T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ)
{
    typedef typename Fast<T>::vec4 vec4;
    __shared__ vec4 tile[256];
    __shared__ T wpart[4];
    __shared__ unsigned long long want[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for_each_molecule_in_range(MACs, n_mols, kMediumMaxAtoms + 1, INT32_MAX, want, nullptr, nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);
        for (int i0 = static_cast<int>(blockIdx.y) * 256; i0 < n; i0 += static_cast<int>(gridDim.y) * 256) {
            const int i = i0 + tid;
            const bool have = i < n;
            const T xi = have ? X[off + i] : T(0), yi = have ? Y[off + i] : T(0), zi = have ? Z[off + i] : T(0),
                    qi = have ? Q[off + i] : T(0);
            T su = T(0), fx = T(0), fy = T(0), fz = T(0);      // sums over j of q_j u and of q_j du (x_i - x_j)
            for (int j0 = 0; j0 < n; j0 += 256) {
                __syncthreads();                               // the previous tile has been used
                const int j = j0 + tid;
                // (places beyond the molecule: charge zero)
                tile[tid] = j < n ? Fast<T>::make4(X[off + j], Y[off + j], Z[off + j], Q[off + j])
                                  : Fast<T>::make4(T(0), T(0), T(0), T(0));
                __syncthreads();
                const int cnt = min(256, n - j0);
#pragma unroll 4
                for (int t = 0; t < cnt; ++t) {
                    const vec4 aj = tile[t];                   // the same address in every lane
                    const T dx = xi - aj.x, dy = yi - aj.y, dz = zi - aj.z;
                    T u, du;
                    pair_terms<T, kDamped>(dx, dy, dz, u, du);      // zero for the atom itself (r = 0)
                    su = fma(aj.w, u, su);
                    if constexpr (kGrad) {
                        const T w = aj.w * du;
                        fx = fma(w, dx, fx);
                        fy = fma(w, dy, fy);
                        fz = fma(w, dz, fz);
                    }
                }
            }
            if (E) {                                           // (the same for every thread)
                const T part = wave_sum(have ? qi * su : T(0));
                __syncthreads();                               // wpart is free
                if (lane == 0) wpart[wave] = part;
                __syncthreads();
                if (tid == 0) atomicAdd(&E[mol], T(0.5) * K * (wpart[0] + wpart[1] + wpart[2] + wpart[3]));
            }
            if (kGrad && have) {
                const T gK = grads[mol] * K;
                if (q_grads) q_grads[off + i] = gK * su;
                if (gX) {
                    gX[off + i] = gK * qi * fx;
                    gY[off + i] = gK * qi * fy;
                    gZ[off + i] = gK * qi * fz;
                }
            }
        }
        __syncthreads();
    });
}

// grid of charge_large_kernel: x = molecules in flight, y = workgroups that share a molecule's blocks of 256 atoms
static dim3 charge_large_grid(int32_t n_mols)
{
    const unsigned columns = static_cast<unsigned>(n_mols < 256 ? n_mols : 256);
    const unsigned parts = columns >= 256 ? 4u : (1024u / columns > 256u ? 256u : 1024u / columns);
    return dim3(columns, parts);
}

}  // namespace

template <typename T>
hipError_t launch_charge_energy(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                                const int32_t* MACs, int32_t n_mols, bool damped, T K, T* E, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + 3u) / 4u;
    // molecules of 65..256 atoms are the tile kernel's, everything else the first kernel's (each leaves the other's alone)
    const unsigned tile_blocks = static_cast<unsigned>(n_mols < 8192 ? n_mols : 8192);
    if (damped) {
        charge_energy_kernel<T, true><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, K, E);
        charge_tile_kernel<T, true, false><<<dim3(tile_blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, nullptr, K, E,
                                                                                   nullptr, nullptr, nullptr, nullptr);
        charge_large_kernel<T, true, false><<<charge_large_grid(n_mols), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, nullptr, K,
                                                                                             E, nullptr, nullptr, nullptr, nullptr);
    } else {
        charge_energy_kernel<T, false><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, K, E);
        charge_tile_kernel<T, false, false><<<dim3(tile_blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, nullptr, K, E,
                                                                                    nullptr, nullptr, nullptr, nullptr);
        charge_large_kernel<T, false, false><<<charge_large_grid(n_mols), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, nullptr, K,
                                                                                              E, nullptr, nullptr, nullptr, nullptr);
    }
    return hipGetLastError();
}

template <typename T>
hipError_t launch_charge_grad(const T* X, const T* Y, const T* Z, const T* Q, const int32_t* MOs,
                              const int32_t* MACs, int32_t n_mols, const T* grads, bool damped, T K, T* q_grads,
                              T* gX, T* gY, T* gZ, T* E, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + 3u) / 4u;
    const unsigned tile_blocks = static_cast<unsigned>(n_mols < 8192 ? n_mols : 8192);
    if (damped) {
        charge_grad_kernel<T, true><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K, q_grads, gX, gY, gZ, E);
        charge_tile_kernel<T, true, true><<<dim3(tile_blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K, E,
                                                                                  q_grads, gX, gY, gZ);
        charge_large_kernel<T, true, true><<<charge_large_grid(n_mols), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K,
                                                                                            E, q_grads, gX, gY, gZ);
    } else {
        charge_grad_kernel<T, false><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K, q_grads, gX, gY, gZ, E);
        charge_tile_kernel<T, false, true><<<dim3(tile_blocks), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K, E,
                                                                                   q_grads, gX, gY, gZ);
        charge_large_kernel<T, false, true><<<charge_large_grid(n_mols), dim3(256), 0, stream>>>(X, Y, Z, Q, MOs, MACs, n_mols, grads, K,
                                                                                             E, q_grads, gX, gY, gZ);
    }
    return hipGetLastError();
}

template hipError_t launch_charge_energy<float>(const float*, const float*, const float*, const float*, const int32_t*, const int32_t*, int32_t, bool, float, float*, hipStream_t);
template hipError_t launch_charge_energy<double>(const double*, const double*, const double*, const double*, const int32_t*, const int32_t*, int32_t, bool, double, double*, hipStream_t);
template hipError_t launch_charge_grad<float>(const float*, const float*, const float*, const float*, const int32_t*, const int32_t*, int32_t, const float*, bool, float, float*, float*, float*, float*, float*, hipStream_t);
template hipError_t launch_charge_grad<double>(const double*, const double*, const double*, const double*, const int32_t*, const int32_t*, int32_t, const double*, bool, double, double*, double*, double*, double*, double*, hipStream_t);

}  // namespace khan
