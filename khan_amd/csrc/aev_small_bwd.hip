// AEV backward (dL/dxyz) for molecules of up to 64 atoms, float32 and float64: one wavefront per molecule.
//
// Lanes are sorted by atom type as in the forward kernel.  A first sweep over the (centre, partner) pairs,
// 64 per step, counts the angular partners of every atom and does the radial part: a lane owns one pair,
// reads the 16 upstream values of the partner's type from the centre's row, sums g e (f_C' - 2 eta d f_C)
// over the shells, and the pull goes to the partner (one group of lanes at a time, so targets are
// distinct) and, summed over the group with DPP moves, to the centre.  Centres are then taken in order
// of decreasing partner count, in batches of up to four whose partner lists together fill at most the 64
// lanes.  Per batch:
//   stage    the 320 angular upstream values of each centre's row are fetched with full-line loads
//            (issued before the scan, so their latency is covered) and laid out in LDS by type pair;
//   scan     64 (centre, partner) pairs per step; angular partners (unit vector, distance, f_C, f_C')
//            go to one pooled list, centre after centre;
//   angular  lane = one list entry (centre b, partner j).  It walks the other partners of the same
//            centre in round-robin order, k = j+1, j+2, ... (mod m): in every round all lanes of a
//            centre hold distinct j AND distinct k, each unordered pair {j,k} is met exactly once.
//            A lane computes its triple completely (32 upstream values from the staged block, three
//            weighted sums formed serially, no cross-lane reduction), keeps the force on j in
//            registers and adds the force on k to slot k of the pooled list with a plain
//            read-add-write: targets are distinct by construction, so no atomics are needed (float
//            atomics on LDS cost ~190 cycles per wave instruction here);
//   gather   centre by centre, every partner's slot is added to its atom's force, and the centre gets
//            minus the sum (each row's forces add up to zero by translation invariance).
// Finally every lane stores the gradient of its own atom: no global atomics, no pre-zeroed output.
// The derivative is the algebraically reduced form (no acos, no 1/(1+cos) factor); reference:
// gpu_featurizer/kernel_cpu.cpp:217-366.
#include "aev_bwd_batch.h"

namespace khan {

namespace {

// centres per batch: four.  Six would fill the pools of 64 entries better (8 % fewer rounds), but the staged upstream
// rows are most of the working set: with four it is 10.2 KB (float) or 20.4 KB (double) and sixteen (eight) wavefronts
// share a CU instead of twelve (six), which is worth more (organic molecules: float 0.68 -> 0.63 ms, double 0.53 -> 0.44 ms).
template <typename T> constexpr int kSmallBwdCentres = 4;

template <typename T>
struct __align__(16) BwdLds {
    typename Fast<T>::vec4 atom[64];     // x, y, z of the atom at this sorted position; w = its type + 4 * (the sorted position of the atom whose index in the molecule is this slot's)
    BwdPool<T, kSmallBwdCentres<T>> pool;   // partner lists and staged upstream values of the batch
    T force[3][64];                      // dL/dx, dL/dy, dL/dz per sorted atom
    int nM[8];                           // angular partners per centre of the batch
};

// float: 4 wavefronts per SIMD (LDS 10.2 KB, 127 registers); double: 2 (LDS 20.4 KB, twice the registers)
template <typename T>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? 4 : 2, sizeof(T) == 4 ? 4 : 2)))
void aev_bwd_small_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<const T> gin, T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ, int max_atoms,
    const int32_t* __restrict__ order)
{
    typedef typename Fast<T>::vec4 vec4;
    __shared__ BwdLds<T> S;
    const int lane = threadIdx.x;
    if (static_cast<int>(blockIdx.x) >= n_mols) return;
    const int mol = order ? uniform(order[blockIdx.x]) : static_cast<int>(blockIdx.x);   // largest first when ordered
    const int n = uniform(MACs[mol]);
    const int off = uniform(MOs[mol]);
    if (n <= 0 || n > max_atoms) return;          // larger molecules belong to other kernels (max_atoms <= 64)
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
        rowbits = reinterpret_cast<unsigned long long>(gin.p[type] + (kOneUpstreamRow ? size_t(0) : static_cast<size_t>(SIs[off + lane]) * kFeats));
    }
    int tcount[4], tbase[4];
    int dest = lane;
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
    S.atom[lane] = Fast<T>::make4(x, y, z, static_cast<T>(type + 4 * dest));     // dest: where the atom with index `lane` went
    S.force[0][lane] = T(0);
    S.force[1][lane] = T(0);
    S.force[2][lane] = T(0);
    auto row_of_lane = [&](int sorted_lane) -> const T* {     // per-lane source index
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(sorted_lane << 2, rp_lo));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(sorted_lane << 2, rp_hi));
        return reinterpret_cast<const T*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };
    auto row_of = [&](int sorted_lane) -> const T* {          // wave-uniform source index
        const unsigned lo = static_cast<unsigned>(lane_read(rp_lo, sorted_lane));
        const unsigned hi = static_cast<unsigned>(lane_read(rp_hi, sorted_lane));
        return reinterpret_cast<const T*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };
    const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
    const int W = 1 << logW, G = 64 >> logW;
    const int grp = lane >> logW, jl = lane & (W - 1);
    const unsigned long long sub_mask = low_bits(W) << ((grp * W) & 63);
    const unsigned long long ltg_mask = lt_mask & sub_mask;
    // type of a sorted lane from the type boundaries
    const int tb1 = tbase[1], tb2 = tbase[2], tb3 = tbase[3];
    auto type_of = [&](int sorted_lane) { return (sorted_lane >= tb1) + (sorted_lane >= tb2) + (sorted_lane >= tb3); };
    wave_lds_fence();
    const vec4 aj = S.atom[jl];      // the partner this lane tests in every scan step
    const int aj_type = static_cast<int>(aj.w) & 3;

    // ------------------------------------------------------------ order of the centres
    // Angular partner count of every atom, then centres in order of decreasing count: a batch of
    // centres shares the lanes of the round-robin walk and runs as long as its busiest centre, so
    // centres with similar counts go together and a batch is cut where its lists fill the 64 lanes.
    int cord, m_at;     // lane p: sorted lane of the centre at position p, and its partner count
    {
        int m_mine = 0;
        for (int s0 = 0; s0 < n; s0 += G) {
            const int i = s0 + grp;
            const vec4 ai = S.atom[min(i, 63)];
            const T dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const T r = Fast<T>::sqrt_rn(dx * dx + dy * dy + dz * dz);
            const bool valid = (i < n) && (jl < n) && (jl != i);
            const bool inA = valid && (r < kA_Rc_f) && (r > T(0));     // r = 0: a coincident atom exerts no force
            const int cnt = popc64(wave_ballot(inA) & sub_mask);          // in every lane of the group
            const int got = __builtin_amdgcn_ds_bpermute((((lane - s0) << logW) & 63) << 2, cnt);
            if (lane >= s0 && lane < s0 + G) m_mine = got;

            // ---- radial pairs: this lane's (centre, partner) pair over its shells (float: the nine nearest to r).  Done here, where the
            // centres come G at a time in lane order, and not per batch, whose last step is rarely full.
            const T* grow = row_of_lane(min(i, 63));
            T cfx = T(0), cfy = T(0), cfz = T(0);       // this pair's pull on the centre
            const bool inR = !kSkipRadial && valid && (r < kR_Rc_f) && (r > T(0));
            if (inR) {
                const T sc = bwd_radial_pair<T>(grow, aj_type, r, Fast<T>::rcp(r));   // dE/dr / r
                cfx = sc * dx;
                cfy = sc * dy;
                cfz = sc * dz;
            }
            // partner forces: one group per round, so the targets of a round are distinct atoms
            for (int g = 0; g < G; ++g) {
                if (inR && grp == g) {
                    S.force[0][jl] -= cfx;
                    S.force[1][jl] -= cfy;
                    S.force[2][jl] -= cfz;
                }
            }
            // the W lanes of a group share their centre: sum inside the group, its last lane adds
            cfx = group_sum_to_last_lane(cfx, logW);
            cfy = group_sum_to_last_lane(cfy, logW);
            cfz = group_sum_to_last_lane(cfz, logW);
            if (jl == W - 1 && i < n) {
                S.force[0][i] += cfx;
                S.force[1][i] += cfy;
                S.force[2][i] += cfz;
            }
        }
        const int key = have ? ((m_mine << 6) | (63 - lane)) : -1;
        int rank = 0;
        for (int l = 0; l < n; ++l) rank += (lane_read(key, l) > key) ? 1 : 0;
        if (!have) rank = lane;
        cord = lane_push(rank, lane);
        m_at = lane_push(rank, m_mine);
    }

    for (int c0 = 0, nb = 0; c0 < n; c0 += nb) {
        // centres of this batch: up to kSmallBwdCentres, lists fitting the 64 lanes; pf[b] = first list slot of centre b
        int pf[kB + 1];
        {
            bool open = true;
            int tot = 0;
            nb = 0;
            pf[0] = 0;
#pragma unroll
            for (int k = 0; k < kB; ++k) {
                int m = 0;
                if (open && k < kSmallBwdCentres<T> && c0 + k < n) {
                    m = lane_read(m_at, min(c0 + k, 63));
                    if (k > 0 && tot + m > 64) {
                        open = false;
                        m = 0;
                    } else {
                        ++nb;
                    }
                } else {
                    open = false;
                }
                tot += m;
                pf[k + 1] = tot;
            }
        }
        const int total = pf[kB];
        unsigned overflow = 0;

        // ---- fetch the angular upstream blocks of the batch's rows (80 x 16 bytes per row)
        RowStage<T, kSmallBwdCentres<T>> stage;
        stage.fetch(lane, nb, [&](int b) { return row_of(lane_read(cord, min(c0 + b, 63))); });
        S.pool.facc[lane] = Fast<T>::make4(T(0), T(0), T(0), T(0));
        if (lane < 8) S.nM[lane] = 0;
        wave_lds_fence();

        // ------------------------------------------------ scan steps: G centres x W partners
        for (int b0 = 0; b0 < nb; b0 += G) {
            const int b = b0 + grp;
            const bool centre_ok = b < nb;
            const int cb = centre_ok ? b : 0;
            const int i = __builtin_amdgcn_ds_bpermute(min(c0 + cb, 63) << 2, cord);
            const int base = sel6(cb, pf[0], pf[1], pf[2], pf[3], pf[4], pf[5]);
            const int room = sel6(cb, pf[1], pf[2], pf[3], pf[4], pf[5], pf[6]) - base;
            const vec4 ai = S.atom[i];
            const T dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const T r = Fast<T>::sqrt_rn(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            const bool inA = valid && (r < kA_Rc_f) && (r > T(0));
            const unsigned long long mA = wave_ballot(inA);
            const int cntA = popc64(mA & sub_mask);
            const bool fits = cntA == room;       // the list has the length the first sweep counted
            const T inv = Fast<T>::rcp(r);
            if (inA && fits) {
                const int pos = base + popc64(mA & ltg_mask);
                T fc, dfc;
                Fast<T>::cutoff_grad(r, static_cast<T>(kA_Rc_f), fc, dfc);
                S.pool.nbr[pos] = Fast<T>::make4(dx * inv, dy * inv, dz * inv, r);
                S.pool.nbr_fc[pos] = Fast<T>::make2(fc, dfc);
                S.pool.nbr_idx[pos] = static_cast<unsigned char>(jl);
            }
            if (jl == 0 && centre_ok) S.nM[b] = fits ? cntA : 0;
            {
                const unsigned long long ov = wave_ballot(!fits && jl == 0 && centre_ok);
                for (int g = 0; g < G; ++g)
                    if ((ov >> (g * W)) & 1ull) overflow |= 1u << (b0 + g);
            }
        }

        // ---- the fetched upstream blocks go to LDS
        stage.store(S.pool, lane, nb);
        wave_lds_fence();

        // ------------------------------------------------ angular: lane = list entry (centre, partner j)
        {
            const int4 m03 = *reinterpret_cast<const int4*>(&S.nM[0]);
            const int4 m47 = *reinterpret_cast<const int4*>(&S.nM[4]);
            // a short pool is walked by two or four lanes per entry, which share its rounds
            const int copies = round_copies(total), span = 64 / copies;
            const int entry = lane & (span - 1), copy = lane / span;
            const int b = (entry >= pf[1]) + (entry >= pf[2]) + (entry >= pf[3]) + (entry >= pf[4]) + (entry >= pf[5]);
            const int bs = entry < total ? b : 0;
            const int pb = sel6(bs, pf[0], pf[1], pf[2], pf[3], pf[4], pf[5]);
            const int m = sel6(bs, m03.x, m03.y, m03.z, m03.w, m47.x, m47.y);   // 0 for a centre that did not fit
            const vec4 fall = bwd_angular_rounds<T>(S.pool, entry, copy, copies, (entry < total) && (m > 0), bs, pb, m, type_of);
            // from here on one lane per entry again
            const bool live = (lane < total) && (m > 0);
            const vec4 f = fall;
            const int self = live ? lane : 0;
            // -------------------------------------------- gather: partners get their slot, the centre minus the sum
            const int atom = S.pool.nbr_idx[self];
            // one add-scan over the lanes per component: a centre's list is a run of lanes, its sum the
            // difference of two prefix values (lane b takes centre b's)
            const T px = group_sum_to_last_lane(live ? f.x : T(0), 6);
            const T py = group_sum_to_last_lane(live ? f.y : T(0), 6);
            const T pz = group_sum_to_last_lane(live ? f.z : T(0), 6);
            {
                const int lo = sel6(min(lane, kB - 1), pf[0], pf[1], pf[2], pf[3], pf[4], pf[5]);
                const int hi = sel6(min(lane, kB - 1), pf[1], pf[2], pf[3], pf[4], pf[5], pf[6]);
                const int at_hi = max(hi - 1, 0) << 2, at_lo = max(lo - 1, 0) << 2;
                T sx = lane_fetch(px, at_hi), sy = lane_fetch(py, at_hi), sz = lane_fetch(pz, at_hi);
                const T qx = lane_fetch(px, at_lo), qy = lane_fetch(py, at_lo), qz = lane_fetch(pz, at_lo);
                if (lo > 0) {
                    sx -= qx;
                    sy -= qy;
                    sz -= qz;
                }
                const int i_b = __builtin_amdgcn_ds_bpermute(min(c0 + lane, 63) << 2, cord);
                if (lane < nb && hi > lo) {          // the centres of a batch are distinct atoms
                    S.force[0][i_b] -= sx;
                    S.force[1][i_b] -= sy;
                    S.force[2][i_b] -= sz;
                }
            }
            wave_lds_fence();
            // partners: one centre at a time, so the atoms of a pass are distinct
            for (int bb = 0; bb < nb; ++bb) {
                if (uniform(pf[bb + 1] - pf[bb]) == 0) continue;
                if (live && (bs == bb)) {
                    S.force[0][atom] += f.x;
                    S.force[1][atom] += f.y;
                    S.force[2][atom] += f.z;
                }
                wave_lds_fence();
            }
        }

        // ------------------------------------------------ centres whose list did not match the first sweep
        if (overflow) {
            for (int b = 0; b < nb; ++b) {
                if (overflow & (1u << b)) {
                    const int i_b = lane_read(cord, min(c0 + b, 63));
                    const int i_orig = lane_read(orig, i_b);
                    bwd_center_generic<T>(L, lane, X, Y, Z, A, off, n, i_orig, S.pool.gst, row_of(i_b),
                                              [&](int atom, T fx, T fy, T fz) {
                                                  const int sl = static_cast<int>(S.atom[atom].w) >> 2;
                                                  atomicAdd(&S.force[0][sl], fx);
                                                  atomicAdd(&S.force[1][sl], fy);
                                                  atomicAdd(&S.force[2][sl], fz);
                                              },
                                              false);        // the radial pairs were done in the first sweep
                }
            }
            wave_lds_fence();
        }
    }

    // ------------------------------------------------------------ every lane stores its own atom
    wave_lds_fence();
    if (have) {
        gX[off + orig] = S.force[0][lane];
        gY[off + orig] = S.force[1][lane];
        gZ[off + orig] = S.force[2][lane];
    }
}

}  // namespace

template <typename T>
hipError_t launch_bwd_small(const T* X, const T* Y, const T* Z, const int32_t* A, const int32_t* MOs,
                            const int32_t* MACs, int32_t n_mols, const int32_t* SIs, Buckets<const T> g,
                            T* gX, T* gY, T* gZ, int max_atoms, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    aev_bwd_small_kernel<T><<<dim3(static_cast<unsigned>(n_mols)), dim3(64), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ, max_atoms < 64 ? max_atoms : 64, order);
    return hipGetLastError();
}

template hipError_t launch_bwd_small<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const float>, float*, float*, float*, int, const int32_t*, hipStream_t);
template hipError_t launch_bwd_small<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const double>, double*, double*, double*, int, const int32_t*, hipStream_t);

}  // namespace khan
