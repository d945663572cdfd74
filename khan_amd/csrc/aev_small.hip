// AEV forward for molecules of up to 64 atoms (float32 and float64): one wavefront per molecule.
//
// How one wavefront spends its 64 lanes
//   sort     one atom per lane, lanes reordered by atom type (4-bin counting sort with ballots).  Every
//            neighbour list built in lane order is then type-sorted, so an unordered type pair (a<=b)
//            owns a contiguous block of (j,k) pairs of a centre.
//   scan     centres are taken six at a time.  A scan step tests 64 (centre, partner) pairs at once:
//            4 centres x 16 partners for molecules of up to 16 atoms, 2 x 32 up to 32, 1 x 64 above.
//            Partners inside the radial cutoff go to a (r, f_C) list, partners inside the angular
//            cutoff to a per-centre list of unit vectors, both compacted with ballot + popcount.
//   radial   lanes = (group of 16) x (shell): a group walks one centre's radial list type by type,
//            two entries per trip, and stores 16 finished floats per (centre, type).
//   phase 1  the triples (centre; j<k) of the six centres are enumerated in (centre, type-pair)
//            order, each segment padded to an even length, and dealt one per lane.  A lane computes
//            what depends on the triple alone: the 8 angular factors (1+cos(theta-theta_t))^8 and the
//            4 radial factors 2^-7 f_C f_C exp(-eta (rho-Rs_s)^2).  12 floats go to LDS.
//   phase 2  lanes = (half, theta_t, Rs_s).  The halves take alternate records; a lane reads G_s of its
//            record (and, in float, one A_t per four records, shared inside its quad) and does one FMA
//            into a register.  Segment boundaries are a bit mask
//            held in scalar registers; at a boundary the halves are added and 32 floats are stored
//            straight to the row in HBM.  Segments without triples are cleared by their lanes of the
//            segment table.
// No atomics and no pre-zeroed output.  A centre with more than 32 angular neighbours (the 3.1 A
// sphere holds about 25 atoms at the densest packings tested) is redone by the general-shape
// per-centre routine.  Semantics: gpu_featurizer/kernel_cpu.cpp:406-537.
#include <cstdlib>
#include <cstring>
#include "aev_fwd_batch.h"

namespace khan {

namespace {

// radial list entries a lane takes per trip: each type's entries are padded to a multiple of this (times the
// number of slots), and two measured faster than one, three or four
constexpr int kRadTrip = 2;
// Entries of the radial lists of one scan step.  A group's list has a fixed place for every partner type, each as
// long as the molecule's number of atoms of that type rounded up to a whole trip of the walk: 16 + 4, 32 + 12 or
// 64 + 28 entries per group for 4, 2 or 1 groups.
constexpr int kRadSlots = 96;

// With kJvp the kernel computes the Jacobian-vector product instead (featurize_grad_inverse): every term of
// the forward sums is replaced by its derivative along the per-atom vectors (VX, VY, VZ).
// float: 4 wavefronts per SIMD (LDS 9.8 KB, <= 128 VGPRs; the kernel loses a fifth of its speed at three);
// float kJvp: 3 (<= 168 VGPRs; its LDS, 13.4 KB, lets twelve wavefronts share a CU); double: 2 (LDS 17 KB); double kJvp: 1.
template <typename T, bool kJvp, bool kMatrixPhase2 = false>
__global__ __launch_bounds__(64 * kWavesPerBlock)
__attribute__((amdgpu_waves_per_eu((kJvp && sizeof(T) == 4) ? 3 : (sizeof(T) == 4 ? 4 : 2) / (kJvp ? 2 : 1), (kJvp && sizeof(T) == 4) ? 3 : (sizeof(T) == 4 ? 4 : 2) / (kJvp ? 2 : 1))))
void aev_fwd_small_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    const T* __restrict__ VX, const T* __restrict__ VY, const T* __restrict__ VZ, Buckets<T> out, int max_atoms,
    const int32_t* __restrict__ order)
{
    typedef typename Fast<T>::vec4 vec4;
    typedef typename Fast<T>::vec2 vec2;
    // centres per batch: six; four in the float Jacobian-vector kernel (with kCap below: twelve wavefronts per CU)
    constexpr int kNB = (kJvp && sizeof(T) == 4) ? 4 : kFB;
    // angular partners kept per centre: 32; 28 in the float Jacobian-vector kernel, whose working set then is 13.4 KB
    // and twelve wavefronts share a CU (a centre with more goes to the general routine, as above 32 elsewhere)
    constexpr int kCap = (kJvp && sizeof(T) == 4) ? 28 : kCapA;
    __shared__ FwdWaveLds<T, kJvp, kNB, kRadSlots, kCap> lds_all[kWavesPerBlock];
    const int lane = threadIdx.x & 63;
    const int wave = kWavesPerBlock == 1 ? 0 : uniform(threadIdx.x >> 6);    // a constant LDS base with one wavefront per workgroup
    const int slot = blockIdx.x * kWavesPerBlock + wave;
    if (slot >= n_mols) return;
    const int mol = order ? uniform(order[slot]) : slot;      // largest molecules first when an order is given
    const int n = uniform(MACs[mol]);
    const int off = uniform(MOs[mol]);
    if (n <= 0 || n > max_atoms) return;          // larger molecules belong to other kernels (max_atoms <= 64)
    FwdWaveLds<T, kJvp, kNB, kRadSlots, kCap>& S = lds_all[wave];
    const LaneConsts<T> L = lane_consts<T>(lane);
    const unsigned long long lane_bit = 1ull << lane;
    const unsigned long long lt_mask = lane_bit - 1ull;

    // ------------------------------------------------------------ load, sort lanes by type
    const bool have = lane < n;
    T x = T(0), y = T(0), z = T(0);
    int type = 0, orig = lane;
    unsigned long long rowbits = 0;
    if (have) {
        x = X[off + lane];
        y = Y[off + lane];
        z = Z[off + lane];
        type = fold_type(A[off + lane]);
        rowbits = reinterpret_cast<unsigned long long>(out.p[type] + static_cast<size_t>(SIs[off + lane]) * kFeats);
    }
    T vx = T(0), vy = T(0), vz = T(0);
    if constexpr (kJvp) {
        if (have) {
            vx = VX[off + lane];
            vy = VY[off + lane];
            vz = VZ[off + lane];
        }
    }
    int tcount[4], tbase[4];
    int dest = lane;    // lanes without an atom keep their place, so the map is a permutation
    {
        unsigned long long tmask[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            tmask[a] = wave_ballot(have && type == a);
            tcount[a] = popc64(tmask[a]);
        }
        tbase[0] = 0;
        tbase[1] = tcount[0];
        tbase[2] = tbase[1] + tcount[1];
        tbase[3] = tbase[2] + tcount[2];
        if (have) {
            const unsigned long long mine = type == 0 ? tmask[0] : type == 1 ? tmask[1] : type == 2 ? tmask[2] : tmask[3];
            dest = sel4(type, tbase[0], tbase[1], tbase[2], tbase[3]) + popc64(mine & lt_mask);
        }
    }
    x = lane_push(dest, x);
    y = lane_push(dest, y);
    z = lane_push(dest, z);
    type = lane_push(dest, type);
    orig = lane_push(dest, orig);
    const int rp_lo = lane_push(dest, static_cast<int>(rowbits & 0xffffffffull));
    const int rp_hi = lane_push(dest, static_cast<int>(rowbits >> 32));
    if constexpr (kJvp) {
        vx = lane_push(dest, vx);
        vy = lane_push(dest, vy);
        vz = lane_push(dest, vz);
    }
    auto row_of = [&](int sorted_lane) -> T* {     // sorted_lane is wave-uniform
        const unsigned lo = static_cast<unsigned>(lane_read(rp_lo, sorted_lane));
        const unsigned hi = static_cast<unsigned>(lane_read(rp_hi, sorted_lane));
        return reinterpret_cast<T*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };
    // sorted-order type ranges: partner index p has type a iff tbase[a] <= p < tbase[a] + tcount[a]
    unsigned long long smask[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) smask[a] = (tcount[a] == 0) ? 0ull : (low_bits(tcount[a]) << tbase[a]);

    // scan geometry: G centres x W partners per step
    const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
    const int W = 1 << logW, G = 64 >> logW;
    const int grp = lane >> logW, jl = lane & (W - 1);
    const unsigned long long sub_mask = low_bits(W) << ((grp * W) & 63);
    const unsigned long long ltg_mask = lt_mask & sub_mask;
    // count lanes: lane l < 16 counts partners of type (l & 3) for group (l >> 2)
    const int cl_g = (lane >> 2) & 3, cl_a = lane & 3;
    const bool cl_on = (lane < 16) && (cl_g < G);
    const unsigned long long cl_sub = cl_on ? (low_bits(W) << ((cl_g * W) & 63)) : 0ull;
    const unsigned long long cl_mask =
        cl_on ? ((cl_a == 0 ? smask[0] : cl_a == 1 ? smask[1] : cl_a == 2 ? smask[2] : smask[3]) << ((cl_g * W) & 63)) : 0ull;
    // radial lanes: 16-lane group rg, shell = lane & 15; the group serves centre group rg_g with
    // entry slot rg_s out of rg_ns slots
    const int rg = lane >> 4;
    const int rg_ns = 4 / G;                                   // 1, 2 or 4
    const int rg_g = G == 4 ? rg : G == 2 ? (rg >> 1) : 0;
    const int rg_s = G == 4 ? 0 : G == 2 ? (rg & 1) : rg;
    // Radial lists: type a's entries of a group start at rbase[a] whatever the centre, and the list is cleared before
    // every step, so the walk reads whole trips without asking how many entries a centre has: an entry that was not
    // written has f_C = 0.  A partner's place is rbase[its type] + the number of in-range partners of that type
    // before it in its group.
    const int rad_unit = kRadTrip * rg_ns;
    const int rad_stride = kRadSlots >> (6 - logW);             // entries per group: 24, 48 or 96
    int rbase[4];
    rbase[0] = 0;
#pragma unroll
    for (int a = 1; a < 4; ++a) rbase[a] = rbase[a - 1] + ((tcount[a - 1] + rad_unit - 1) & -rad_unit);
    const int tj = __builtin_amdgcn_ds_bpermute(jl << 2, type);
    const int rad_pos0 = grp * rad_stride + sel4(tj, rbase[0], rbase[1], rbase[2], rbase[3]);
    const unsigned long long rad_mask = lt_mask & (~0ull << ((grp * W + sel4(tj, tbase[0], tbase[1], tbase[2], tbase[3])) & 63));
    // the sorted atoms stay in the lanes' registers: the partner this lane tests in every scan step, once; the
    // step's centres by lane exchange
    const T xj = lane_fetch(x, jl << 2), yj = lane_fetch(y, jl << 2), zj = lane_fetch(z, jl << 2);
    T vxj = T(0), vyj = T(0), vzj = T(0);
    if constexpr (kJvp) {
        vxj = lane_fetch(vx, jl << 2);
        vyj = lane_fetch(vy, jl << 2);
        vzj = lane_fetch(vz, jl << 2);
    }

    fwd_lds_init(S, lane);
    wave_lds_fence();

    for (int c0 = 0; c0 < n; c0 += kNB) {
        const int nb = min(kNB, n - c0);
        unsigned overflow = 0;

        // ------------------------------------------------ scan steps: G centres x W partners
        for (int b0 = 0; b0 < nb; b0 += G) {
            const int b = b0 + grp;                      // centre-in-batch of this lane's group
            const int i = c0 + b;
            const bool centre_ok = b < nb;
            const int ci = (centre_ok ? i : 0) << 2;
            // clears the lists: every lane two entries (the upper half of the wavefront repeats the lower half's second one)
            static_assert(kRadSlots == 96, "64 + 32 entries");
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int at = e == 0 ? lane : 64 + (lane & 31);
                S.rad[at] = Fast<T>::make2(T(0), T(0));
                if constexpr (kJvp) S.jvp.rad_ab[at] = Fast<T>::make2(T(0), T(0));
            }
            const T dx = lane_fetch(x, ci) - xj, dy = lane_fetch(y, ci) - yj, dz = lane_fetch(z, ci) - zj;
            const T r = Fast<T>::sqrt_rn(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            // a coincident atom (r = 0) has no direction: it takes no part in any derivative.  In the features it
            // counts as the reference counts it: its cosine is 0/0, which the clamp turns into -1 (kernel_cpu.cpp:514-516)
            const bool inR = valid && (r < kR_Rc_f) && (!kJvp || r > T(0));
            const bool inA = valid && (r < kA_Rc_f) && (!kJvp || r > T(0));
            const unsigned long long mR = wave_ballot(inR), mA = wave_ballot(inA);
            const bool fits = popc64(mA & sub_mask) <= kCap;
            T wx = T(0), wy = T(0), wz = T(0), rd = T(0);        // v_centre - v_partner, and d r along it
            const T inv = Fast<T>::rcp(r);
            if constexpr (kJvp) {
                // the incoming vectors stay in the lanes like the positions: the partner's once, the centre's by lane exchange
                wx = lane_fetch(vx, ci) - vxj;
                wy = lane_fetch(vy, ci) - vyj;
                wz = lane_fetch(vz, ci) - vzj;
                rd = (dx * wx + dy * wy + dz * wz) * inv;
            }
            if (inR) {
                const int pos = rad_pos0 + popc64(mR & rad_mask);
                if constexpr (kJvp) {
                    T fc, dfc;
                    Fast<T>::cutoff_grad(r, static_cast<T>(kR_Rc_f), fc, dfc);
                    S.rad[pos] = Fast<T>::make2(r, fc);
                    S.jvp.rad_ab[pos] = Fast<T>::make2(dfc * rd, T(-2) * static_cast<T>(kR_eta_f) * fc * rd);
                } else {
                    S.rad[pos] = Fast<T>::make2(r, Fast<T>::cutoff(r, static_cast<T>(kR_Rc_f)));
                }
            }
            if (inA && fits) {
                const int pos = popc64(mA & ltg_mask);
                const int cb = centre_ok ? b : 0;
                S.nbr[cb][pos] = Fast<T>::make4(dx * inv, dy * inv, dz * inv, r);
                if constexpr (kJvp) {
                    T fc, dfc;
                    Fast<T>::cutoff_grad(r, static_cast<T>(kA_Rc_f), fc, dfc);
                    S.nbr_fc[cb][pos] = fc;
                    S.jvp.nbr_p[cb][pos] = Fast<T>::make4(wx * inv, wy * inv, wz * inv, rd * inv);
                    S.jvp.nbr_dfc[cb][pos] = dfc * rd;
                } else {
                    S.nbr_fc[cb][pos] = Fast<T>::cutoff(r, static_cast<T>(kA_Rc_f));
                }
            }
            {   // bit b of `overflow`: centre b of the batch has too many angular partners
                const unsigned long long ov = wave_ballot(!fits && jl == 0 && centre_ok);
                for (int g = 0; g < G; ++g)
                    if ((ov >> (g * W)) & 1ull) overflow |= 1u << (b0 + g);
            }
            int cntR = 0;
            if (cl_on) {
                const int cb = b0 + cl_g;
                cntR = popc64(mR & cl_mask);
                if (cb < nb) S.nA[cb][cl_a] = (popc64(mA & cl_sub) <= kCap) ? popc64(mA & cl_mask) : 0;
            }
            // largest radial count of each type over the groups of this step (lanes 0..15 hold them)
            int mx = cntR;
            mx = max(mx, __builtin_amdgcn_update_dpp(0, mx, 0x124, 0xf, 0xf, false));   // row_ror:4
            mx = max(mx, __builtin_amdgcn_update_dpp(0, mx, 0x128, 0xf, 0xf, false));   // row_ror:8
            const int mxR[4] = {lane_read(mx, 0), lane_read(mx, 1), lane_read(mx, 2), lane_read(mx, 3)};
            wave_lds_fence();

            // ---- radial features of the G centres of this step
            {
                const vec2* list = &S.rad[rg_g * rad_stride + rg_s];
                const int cb = b0 + rg_g;
                const int ci = min(c0 + cb, 63);
                const unsigned rlo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(ci << 2, rp_lo));
                const unsigned rhi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(ci << 2, rp_hi));
                T* row = reinterpret_cast<T*>((static_cast<unsigned long long>(rhi) << 32) | rlo);
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    T acc_r = T(0);
                    const vec2* pl = list + rbase[a];
                    for (int q0 = 0; q0 < (kSkipRadial ? 0 : mxR[a]); q0 += rad_unit) {
                        // kRadTrip entries of this lane's slot per trip; slot s takes q = s, s+ns, s+2ns, ...
                        vec2 e[kRadTrip], ab[kRadTrip];
#pragma unroll
                        for (int u = 0; u < kRadTrip; ++u) {
                            e[u] = pl[q0 + u * rg_ns];
                            if constexpr (kJvp) ab[u] = S.jvp.rad_ab[rg_g * rad_stride + rg_s + rbase[a] + q0 + u * rg_ns];
                        }
#pragma unroll
                        for (int u = 0; u < kRadTrip; ++u) {
                            const T dd = e[u].x - L.rrs;
                            // forward: exp(-eta d^2) f_C; derivative: exp(-eta d^2) (f_C' - 2 eta d f_C) dr
                            const T v = Fast<T>::gauss(static_cast<T>(kR_eta_f), dd);
                            if constexpr (kJvp) acc_r = fma(v, fma(ab[u].y, dd, ab[u].x), acc_r);
                            else acc_r = fma(v, e[u].y, acc_r);
                        }
                    }
                    if (rg_ns >= 2) acc_r += __shfl_xor(acc_r, 16, 64);
                    if (rg_ns == 4) acc_r += __shfl_xor(acc_r, 32, 64);
                    if (rg_s == 0 && cb < nb) store_global(row + a * kNumRRs + (lane & 15), acc_r);
                }
            }
            wave_lds_fence();
        }

        // ------------------------------------------------ segment table, phases 1 and 2, zero fill
        fwd_angular_batch<kMatrixPhase2>(S, L, lane, nb, [&](int b) -> unsigned long long {
            const int cl = min(c0 + b, 63);
            const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(cl << 2, rp_lo));
            const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(cl << 2, rp_hi));
            return (static_cast<unsigned long long>(hi) << 32) | lo;
        });

        // ------------------------------------------------ centres whose list overflowed
        if (overflow) {
            __threadfence();
            for (int b = 0; b < nb; ++b) {
                if (overflow & (1u << b)) {
                    const int i_orig = lane_read(orig, c0 + b);
                    if constexpr (kJvp)
                        jvp_center_generic<T>(L, lane, X, Y, Z, A, VX, VY, VZ, off, n, i_orig,
                                              reinterpret_cast<T*>(S.rec), row_of(c0 + b));
                    else
                        fwd_center_generic<T>(L, lane, X, Y, Z, A, off, n, i_orig,
                                              reinterpret_cast<T*>(S.rec), row_of(c0 + b));
                }
            }
            wave_lds_fence();
        }
    }
}

}  // namespace

template <typename T>
hipError_t launch_fwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<T> out,
                            int max_atoms, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kWavesPerBlock - 1u) / kWavesPerBlock;
#ifdef KHAN_CHECK_BUILD
    if constexpr (sizeof(T) == 4) {
        // check build only: KHAN_AEV_PHASE2=matrix (read once) selects the variant that sums the angular records on the
        // matrix cores; it is slower than the default and kept for measurement
        static const bool matrix_phase2 = [] {
            const char* v = std::getenv("KHAN_AEV_PHASE2");
            return v != nullptr && std::strcmp(v, "matrix") == 0;
        }();
        if (matrix_phase2) {
            aev_fwd_small_kernel<T, false, true><<<dim3(blocks), dim3(64 * kWavesPerBlock), 0, stream>>>(
                X, Y, Z, A, MOs, MACs, n_mols, SIs, nullptr, nullptr, nullptr, out, max_atoms < 64 ? max_atoms : 64, order);
            return hipGetLastError();
        }
    }
#endif
    aev_fwd_small_kernel<T, false><<<dim3(blocks), dim3(64 * kWavesPerBlock), 0, stream>>>(
        X, Y, Z, A, MOs, MACs, n_mols, SIs, nullptr, nullptr, nullptr, out, max_atoms < 64 ? max_atoms : 64, order);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_jvp_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, const T* VX,
                            const T* VY, const T* VZ, Buckets<T> out, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kWavesPerBlock - 1u) / kWavesPerBlock;
    aev_fwd_small_kernel<T, true><<<dim3(blocks), dim3(64 * kWavesPerBlock), 0, stream>>>(
        X, Y, Z, A, MOs, MACs, n_mols, SIs, VX, VY, VZ, out, kSmallMaxAtoms, order);
    return hipGetLastError();
}

template hipError_t launch_fwd_small<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<float>, int, const int32_t*, hipStream_t);
template hipError_t launch_fwd_small<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<double>, int, const int32_t*, hipStream_t);
template hipError_t launch_jvp_small<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const float*, const float*, const float*, Buckets<float>, const int32_t*, hipStream_t);
template hipError_t launch_jvp_small<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const double*, const double*, const double*, Buckets<double>, const int32_t*, hipStream_t);

}  // namespace khan
