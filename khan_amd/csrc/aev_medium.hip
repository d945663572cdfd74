// AEV forward for molecules of up to 256 atoms that are too large for one wavefront (float32 from 33 atoms,
// float64 from 65; also the float32 Jacobian-vector product from 65): one workgroup of four wavefronts per molecule.
//
// The workgroup sorts the molecule's atoms by type into LDS once (256-way counting sort with per-wave
// ballots).  Each wavefront then takes batches of four or six centres (see kNB below) and runs the same pipeline as the
// one-wavefront-per-molecule kernel on them:
//   scan     a centre is tested against the sorted atoms 64 at a time; partners inside the radial
//            cutoff are appended to a (r, f_C) list, partners inside the angular cutoff to the centre's
//            list of unit vectors.  Chunks are consecutive ranges of the sorted order, so both lists
//            stay sorted by type.
//   radial   lanes = (slot of 4) x (shell): a centre's list is walked type by type, four entries per
//            trip, and 16 finished floats per type go straight to the row.
//   angular  segment table, triple-per-lane factors and the (theta_t, Rs_s) accumulation of the shared
//            batch routine.
// Rows are written once, without atomics.  A centre with more than 32 angular or 64 radial partners is
// redone by the general per-centre routine.  Semantics: gpu_featurizer/kernel_cpu.cpp:406-537.
#include "aev_fwd_batch.h"
#include "aev_large.h"

namespace khan {

namespace {

constexpr int kRadCap = 64;                   // radial partners kept per centre
constexpr int kMedRadTrip = 1;                // list entries a lane takes per trip of the radial walk (four slots: 4 entries per trip)

template <typename T, bool kJvp> struct MedVel {};
template <typename T> struct __align__(16) MedVel<T, true> {
    typename Fast<T>::vec4 vel[kMediumMaxAtoms];   // the incoming vector of every atom (sorted order)
};

template <typename T, bool kJvp, bool kLarge = false>
struct __align__(16) MedShared {
    typename Fast<T>::vec4 atom[kMediumMaxAtoms];   // x, y, z, type (sorted order)
    unsigned row_lo[kMediumMaxAtoms];      // address of the atom's output row
    unsigned row_hi[kMediumMaxAtoms];
    unsigned short orig[kMediumMaxAtoms];  // sorted position -> index inside the molecule
    int wcount[4][4];                      // atoms of each type held by each wavefront before the sort
    MedVel<T, kJvp> v;
};
// above 256 atoms the sorted atoms are in device memory (aev_large.h); what stays here are the output rows of the
// centres of each wavefront's batch
template <typename T, bool kJvp>
struct __align__(16) MedShared<T, kJvp, true> {
    unsigned long long row[4][8];
    // partner types of the entries of each wavefront's radial list and of the angular list it is building (used by the
    // Jacobian-vector product, whose list entries have no room for the type)
    unsigned char rtype[4][kRadCap];
    unsigned char atype[4][kCapA];
};

// With kJvp the kernel computes the Jacobian-vector product instead (featurize_grad_inverse), as the
// one-wavefront kernel does: list entries also carry (v_i - v_j)/r, the cutoff's derivative and the change of r.
// With kLarge the kernel takes the molecules of more than 256 atoms: the atoms come type-sorted from `sorted`, and
// the workgroups of one grid column (blockIdx.y = 0 .. gridDim.y - 1) share a molecule's centres batch by batch.
template <typename T, bool kJvp, bool kLarge = false>
__global__ __launch_bounds__(256) void aev_fwd_medium_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    const T* __restrict__ VX, const T* __restrict__ VY, const T* __restrict__ VZ,
    Buckets<T> out, int min_atoms, const int32_t* __restrict__ order, const SortedAtoms<T> sorted)
{
    typedef typename Fast<T>::vec4 vec4;
    typedef typename Fast<T>::vec2 vec2;
    __shared__ MedShared<T, kJvp, kLarge> M;
    // Batches of four centres in float32: the forward kernel's working set then lets four workgroups share a CU
    // (LDS 39.9 KB each) instead of three, which measured 21 % faster on dense boxes, and the Jacobian-vector kernel's
    // two (75 KB each) instead of one; the float64 forward kernel keeps batches of six, and the float64 Jacobian-vector
    // kernel takes batches of four (134 KB, one workgroup per CU; six measured the same at 157 KB of the CU's 160).
    constexpr int kNB = (sizeof(T) == 4 || kJvp) ? 4 : kFB;
    __shared__ FwdWaveLds<T, kJvp, kNB> lds_wave[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    FwdWaveLds<T, kJvp, kNB>& S = lds_wave[wave];
    const LaneConsts<T> L = lane_consts<T>(lane);
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    const int rslot = lane >> 4;                                 // radial walk: entry slot of this 16-lane group

    fwd_lds_init(S, lane);
    __shared__ unsigned long long want[4];
    for_each_molecule_in_range(MACs, n_mols, min_atoms, kLarge ? INT32_MAX : kMediumMaxAtoms, want, order, order ? order + n_mols : nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);

        // ------------------------------------------------------------ load, sort by type into LDS
        if constexpr (!kLarge) {
        const bool have = tid < n;
        T x = T(0), y = T(0), z = T(0);
        T vx = T(0), vy = T(0), vz = T(0);
        int type = 0;
        unsigned long long rowbits = 0;
        if (have) {
            x = X[off + tid];
            y = Y[off + tid];
            z = Z[off + tid];
            type = fold_type(A[off + tid]);
            rowbits = reinterpret_cast<unsigned long long>(out.p[type] + static_cast<size_t>(SIs[off + tid]) * kFeats);
            if constexpr (kJvp) {
                vx = VX[off + tid];
                vy = VY[off + tid];
                vz = VZ[off + tid];
            }
        }
        unsigned long long tmask[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) tmask[a] = wave_ballot(have && type == a);
        if (lane < 4) M.wcount[wave][lane] = popc64(lane == 0 ? tmask[0] : lane == 1 ? tmask[1] : lane == 2 ? tmask[2] : tmask[3]);
        __syncthreads();
        int tbase[4], tcount[4];
        {
            int run = 0;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                tbase[a] = run;
                tcount[a] = M.wcount[0][a] + M.wcount[1][a] + M.wcount[2][a] + M.wcount[3][a];
                run += tcount[a];
            }
        }
        if (have) {
            int before = 0;                     // atoms of my type held by earlier wavefronts
            for (int w = 0; w < wave; ++w) before += M.wcount[w][type];
            const unsigned long long mine = type == 0 ? tmask[0] : type == 1 ? tmask[1] : type == 2 ? tmask[2] : tmask[3];
            const int dest = sel4(type, tbase[0], tbase[1], tbase[2], tbase[3]) + before + popc64(mine & lt_mask);
            M.atom[dest] = Fast<T>::make4(x, y, z, static_cast<T>(type));
            M.row_lo[dest] = static_cast<unsigned>(rowbits & 0xffffffffull);
            M.row_hi[dest] = static_cast<unsigned>(rowbits >> 32);
            M.orig[dest] = static_cast<unsigned short>(tid);
            if constexpr (kJvp) M.v.vel[dest] = Fast<T>::make4(vx, vy, vz, T(0));
        }
        __syncthreads();
        }
        const int last_atom = (kLarge ? n : kMediumMaxAtoms) - 1;
        const int n_chunks = (n + 63) >> 6;
        const size_t chunk0 = kLarge ? chunk_base(off, mol) : 0;     // the molecule's first chunk box
        auto atom_at = [&](int sorted_idx) -> vec4 {
            if constexpr (kLarge) return sorted.atom[off + sorted_idx];
            else return M.atom[sorted_idx];
        };
        auto vel_at = [&](int sorted_idx) -> vec4 {
            if constexpr (!kJvp) return Fast<T>::make4(T(0), T(0), T(0), T(0));
            else if constexpr (kLarge) return sorted.vel[off + sorted_idx];
            else return M.v.vel[sorted_idx];
        };
        auto orig_of = [&](int sorted_idx) -> int {          // wave-uniform index
            if constexpr (kLarge) return uniform(sorted.aux[off + sorted_idx].x);
            else return uniform(static_cast<int>(M.orig[sorted_idx]));
        };
        int c0 = 0;                                          // first centre of the wavefront's batch
        auto row_bits_of = [&](int sorted_idx) -> unsigned long long {     // per-lane index inside the batch's range
            if constexpr (kLarge) {
                return M.row[wave][min(max(sorted_idx - c0, 0), 7)];
            } else {
                const int idx = min(sorted_idx, kMediumMaxAtoms - 1);
                return (static_cast<unsigned long long>(M.row_hi[idx]) << 32) | M.row_lo[idx];
            }
        };
        auto row_of = [&](int sorted_idx) -> T* {            // wave-uniform index
            const unsigned long long bits = row_bits_of(sorted_idx);
            const unsigned lo = static_cast<unsigned>(uniform(static_cast<int>(bits & 0xffffffffull)));
            const unsigned hi = static_cast<unsigned>(uniform(static_cast<int>(bits >> 32)));
            return reinterpret_cast<T*>((static_cast<unsigned long long>(hi) << 32) | lo);
        };

        // ------------------------------------------------------------ batches of kNB centres per wavefront
        // (a large molecule that has the grid column to itself: shorter batches, so that every wavefront gets centres)
        const int waves_y = static_cast<int>(gridDim.y) * 4;
        const int batch = kLarge ? max(1, min(kNB, (n + waves_y - 1) / waves_y)) : kNB;
        const int first_c0 = (kLarge ? static_cast<int>(blockIdx.y) * 4 + wave : wave) * batch;
        const int stride_c0 = (kLarge ? waves_y : 4) * batch;
        for (c0 = first_c0; c0 < n; c0 += stride_c0) {
            const int nb = min(batch, n - c0);
            unsigned overflow = 0;
            if constexpr (kLarge) {
                if (lane < nb) {
                    const int type = static_cast<int>(sorted.atom[off + c0 + lane].w);
                    T* const bucket = type == 0 ? out.p[0] : type == 1 ? out.p[1] : type == 2 ? out.p[2] : out.p[3];
                    M.row[wave][lane] = reinterpret_cast<unsigned long long>(bucket + static_cast<size_t>(sorted.aux[off + c0 + lane].y) * kFeats);
                }
                wave_lds_fence();
            }

            for (int b = 0; b < nb; ++b) {
                const int i = c0 + b;
                const vec4 ai = atom_at(i);
                int posR = 0, posA = 0;                 // list lengths so far (wave-uniform)
                int cR[4] = {0, 0, 0, 0}, cA[4] = {0, 0, 0, 0};
                // adds the radial list's entries (cnt[a] of type a, laid end to end) to acc[a]: lanes = (slot of 4) x (shell)
                auto radial_sums = [&](T (&acc)[4], const int (&cnt)[4]) {
                    int obase = 0;
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const int cnt_a = cnt[a];
                        T acc_r = T(0);
                        for (int q0 = 0; q0 < (kSkipRadial ? 0 : cnt_a); q0 += 4 * kMedRadTrip) {
                            vec2 e[kMedRadTrip], ab[kMedRadTrip];
#pragma unroll
                            for (int u = 0; u < kMedRadTrip; ++u) {
                                const int at = min(obase + q0 + u * 4 + rslot, kRadCap - 1);
                                e[u] = S.rad[at];
                                if constexpr (kJvp) ab[u] = S.jvp.rad_ab[at];
                            }
#pragma unroll
                            for (int u = 0; u < kMedRadTrip; ++u) {
                                const T dd = e[u].x - L.rrs;
                                // forward: exp(-eta d^2) f_C; derivative: exp(-eta d^2) (f_C' - 2 eta d f_C) dr
                                T v = Fast<T>::gauss(static_cast<T>(kR_eta_f), dd);
                                if constexpr (kJvp) v *= fma(ab[u].y, dd, ab[u].x);
                                else v *= e[u].y;
                                acc_r += (q0 + u * 4 + rslot < cnt_a) ? v : T(0);   // entries of other types: select
                            }
                        }
                        acc[a] += acc_r;
                        obase += cnt_a;
                    }
                };
                // Large molecules: a centre's radial list is worked off whenever the next chunk's entries would not fit
                // (no limit on the number of radial partners); racc collects the sums.
                T racc[4] = {T(0), T(0), T(0), T(0)};
                auto radial_flush = [&](int count) {
                    wave_lds_fence();
                    // the entries arrive in the order of the sorted atoms (by cell): put them in order of type
                    int tR = -1;
                    vec2 e = Fast<T>::make2(T(0), T(0)), ab = Fast<T>::make2(T(0), T(0));
                    if (lane < count) {
                        e = S.rad[lane];
                        if constexpr (kJvp) ab = S.jvp.rad_ab[lane];
                        if constexpr (kJvp && kLarge) tR = M.rtype[wave][lane];
                        else tR = static_cast<int>(e.y);
                    }
                    int cnt[4], dest = 0, before = 0;
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const unsigned long long ma = wave_ballot(tR == a);
                        cnt[a] = popc64(ma);
                        if (tR == a) dest = before + popc64(ma & lt_mask);
                        before += cnt[a];
                    }
                    wave_lds_fence();               // every entry has been read
                    if (lane < count) {
                        if constexpr (kJvp) {
                            S.rad[dest] = e;
                            S.jvp.rad_ab[dest] = ab;
                        } else {
                            S.rad[dest] = Fast<T>::make2(e.x, Fast<T>::cutoff(e.x, static_cast<T>(kR_Rc_f)));
                        }
                    }
                    wave_lds_fence();
                    radial_sums(racc, cnt);
                    wave_lds_fence();               // the list may be overwritten
                };
                // one chunk of 64 partners: aj (and with kJvp vjv) of the atom at sorted position jc + lane
                auto scan_chunk = [&](int jc, const vec4 aj, const vec4 vjv) {
                    const int j = jc + lane;
                    const T dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
                    const T r = Fast<T>::sqrt_rn(dx * dx + dy * dy + dz * dz);
                    const bool valid = (j < n) && (j != i);
                    // r = 0, a coincident atom: no part in derivatives; in the features as the reference has it
                    const bool inR = valid && (r < kR_Rc_f) && (!kJvp || r > T(0));
                    const bool inA = valid && (r < kA_Rc_f) && (!kJvp || r > T(0));
                    const unsigned long long mR = wave_ballot(inR), mA = wave_ballot(inA);
                    if constexpr (kLarge) {
                        if (posR + popc64(mR) > kRadCap) {
                            radial_flush(posR);
                            posR = 0;
                        }
                    }
                    if constexpr (kJvp) {
                        const int tj = static_cast<int>(aj.w);
#pragma unroll
                        for (int a = 0; a < 4; ++a) {
                            const unsigned long long ta = wave_ballot(tj == a);
                            cR[a] += popc64(mR & ta);
                            cA[a] += popc64(mA & ta);
                        }
                        const T inv = Fast<T>::rcp(r);
                        const vec4 vi = vel_at(i);
                        const T wx = vi.x - vjv.x, wy = vi.y - vjv.y, wz = vi.z - vjv.z;     // v_centre - v_partner
                        const T rd = (dx * wx + dy * wy + dz * wz) * inv;                    // d r along it
                        if (inR) {
                            const int p = posR + popc64(mR & lt_mask);
                            if (p < kRadCap) {
                                T fc, dfc;
                                Fast<T>::cutoff_grad(r, static_cast<T>(kR_Rc_f), fc, dfc);
                                S.rad[p] = Fast<T>::make2(r, fc);
                                S.jvp.rad_ab[p] = Fast<T>::make2(dfc * rd, T(-2) * static_cast<T>(kR_eta_f) * fc * rd);
                                if constexpr (kLarge) M.rtype[wave][p] = static_cast<unsigned char>(tj);
                            }
                        }
                        if (inA) {
                            const int p = posA + popc64(mA & lt_mask);
                            if (p < kCapA) {
                                T fc, dfc;
                                Fast<T>::cutoff_grad(r, static_cast<T>(kA_Rc_f), fc, dfc);
                                S.nbr[b][p] = Fast<T>::make4(dx * inv, dy * inv, dz * inv, r);
                                S.nbr_fc[b][p] = fc;
                                S.jvp.nbr_p[b][p] = Fast<T>::make4(wx * inv, wy * inv, wz * inv, rd * inv);
                                S.jvp.nbr_dfc[b][p] = dfc * rd;
                                if constexpr (kLarge) M.atype[wave][p] = static_cast<unsigned char>(tj);
                            }
                        }
                    } else {
                        // Only a fraction of a chunk's atoms lies inside the cutoffs: the chunk stores what it found
                        // as it is (distance; difference vector), and the cutoff functions and unit vectors are
                        // worked out once per centre on the compacted lists below, not once per chunk on every lane.
                        // (the place of the cutoff value carries the partner's type until then)
                        if (inR) {
                            const int p = posR + popc64(mR & lt_mask);
                            if (p < kRadCap) S.rad[p] = Fast<T>::make2(r, aj.w);
                        }
                        if (inA) {
                            const int p = posA + popc64(mA & lt_mask);
                            if (p < kCapA) {
                                S.nbr[b][p] = Fast<T>::make4(dx, dy, dz, r);
                                S.nbr_fc[b][p] = aj.w;
                            }
                        }
                    }
                    posR += popc64(mR);
                    posA += popc64(mA);
                };
                if constexpr (kLarge) {
                    // From device memory.  The atoms are sorted by type and, inside a type, along a space-filling
                    // curve: 64 chunks' boxes are tested against the centre at a time (one per lane), and only the
                    // chunks that reach into the radial cutoff are scanned, four chunks' loads in flight at a time.
                    const float cx = static_cast<float>(ai.x), cy = static_cast<float>(ai.y), cz = static_cast<float>(ai.z);
                    for (int ch0 = 0; ch0 < n_chunks; ch0 += 64) {
                        unsigned long long near = wave_ballot(chunk_in_reach(sorted.box + 2 * chunk0, ch0 + lane, n_chunks, cx, cy, cz));
                        while (near) {
                            int ch[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                ch[u] = -1;
                                if (near) {
                                    ch[u] = ch0 + lowest_bit(near);
                                    near &= near - 1;
                                }
                            }
                            vec4 at[4], vt[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                const int jj = min(max(ch[u], 0) * 64 + lane, last_atom);
                                at[u] = atom_at(jj);
                                vt[u] = vel_at(jj);
                            }
#pragma unroll
                            for (int u = 0; u < 4; ++u)
                                if (ch[u] >= 0) scan_chunk(ch[u] * 64, at[u], vt[u]);
                        }
                    }
                } else {
                    for (int jc = 0; jc < n; jc += 64) {
                        const int jj = min(jc + lane, last_atom);
                        scan_chunk(jc, atom_at(jj), vel_at(jj));
                    }
                }
                if constexpr (kLarge) {
                    radial_flush(posR);
                    // the angular list too arrives in the order of the sorted atoms: put it in order of type
                    const bool haveE = lane < min(posA, kCapA);
                    int tA = -1;
                    vec4 nb = Fast<T>::make4(T(0), T(0), T(0), T(0)), np = nb;
                    T nd = T(0);
                    T fc = T(0);
                    if (haveE) {
                        nb = S.nbr[b][lane];
                        fc = S.nbr_fc[b][lane];
                        if constexpr (kJvp) {
                            np = S.jvp.nbr_p[b][lane];
                            nd = S.jvp.nbr_dfc[b][lane];
                            tA = M.atype[wave][lane];
                        } else {
                            tA = static_cast<int>(fc);
                        }
                    }
                    int dest = 0, before = 0;
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const unsigned long long ma = wave_ballot(tA == a);
                        if (tA == a) dest = before + popc64(ma & lt_mask);
                        before += popc64(ma);
                    }
                    wave_lds_fence();               // every entry has been read
                    if (haveE) {
                        S.nbr[b][dest] = nb;
                        S.nbr_fc[b][dest] = fc;
                        if constexpr (kJvp) {
                            S.jvp.nbr_p[b][dest] = np;
                            S.jvp.nbr_dfc[b][dest] = nd;
                        }
                    }
                }
                if constexpr (!kJvp) {
                    wave_lds_fence();
                    const bool haveR = !kLarge && lane < min(posR, kRadCap), haveA = lane < min(posA, kCapA);
                    int tR = -1, tA = -1;           // type of this lane's list entry
                    if (haveR) {
                        const vec2 e = S.rad[lane];
                        tR = static_cast<int>(e.y);
                        S.rad[lane] = Fast<T>::make2(e.x, Fast<T>::cutoff(e.x, static_cast<T>(kR_Rc_f)));
                    }
                    if (haveA) {
                        const vec4 d = S.nbr[b][lane];
                        tA = static_cast<int>(S.nbr_fc[b][lane]);
                        const T inv = Fast<T>::rcp(d.w);
                        S.nbr[b][lane] = Fast<T>::make4(d.x * inv, d.y * inv, d.z * inv, d.w);
                        S.nbr_fc[b][lane] = Fast<T>::cutoff(d.w, static_cast<T>(kA_Rc_f));
                    }
                    // partners per type, from the compacted lists (once per centre; lists that overflowed are redone
                    // by the general routine and their counts are not used)
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        cR[a] = popc64(wave_ballot(tR == a));
                        cA[a] = popc64(wave_ballot(tA == a));
                    }
                }
                const bool fits = (kLarge || posR <= kRadCap) && (posA <= kCapA);
                if (!fits) overflow |= 1u << b;
                if (lane < 4) S.nA[b][lane] = fits ? sel4(lane, cA[0], cA[1], cA[2], cA[3]) : 0;
                wave_lds_fence();

                // ---- radial features of this centre: lanes = (slot of 4) x (shell)
                if (fits) {
                    T* row = row_of(i);
                    T acc[4] = {racc[0], racc[1], racc[2], racc[3]};
                    if constexpr (!kLarge) radial_sums(acc, cR);
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        T acc_r = acc[a];
                        acc_r += __shfl_xor(acc_r, 16, 64);
                        acc_r += __shfl_xor(acc_r, 32, 64);
                        if (rslot == 0) store_global(row + a * kNumRRs + (lane & 15), acc_r);
                    }
                }
                wave_lds_fence();
            }

            // ------------------------------------------------ segment table, phases 1 and 2, zero fill
            fwd_angular_batch<false>(S, L, lane, nb, [&](int b) -> unsigned long long { return row_bits_of(c0 + b); });

            // ------------------------------------------------ centres whose lists overflowed
            if (overflow) {
                __threadfence();
                for (int b = 0; b < nb; ++b) {
                    if (overflow & (1u << b)) {
                        const int i_orig = orig_of(c0 + b);
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
        __syncthreads();      // the next molecule reuses the sorted arrays
    });
}

}  // namespace

template <typename T>
hipError_t launch_fwd_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, Buckets<T> out, int min_atoms, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    // workgroups walk the molecules with the grid's stride and skip those of other sizes
    // (in float64 the working set lets one workgroup run per CU: a smaller grid costs less when it only skips)
    const int32_t cap = sizeof(T) == 4 ? 4096 : 1024;
    const unsigned blocks = static_cast<unsigned>(n_mols < cap ? n_mols : cap);
    aev_fwd_medium_kernel<T, false><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, nullptr, nullptr,
                                                                        nullptr, out, min_atoms, order, SortedAtoms<T>{});
    return hipGetLastError();
}

template <typename T>
hipError_t launch_jvp_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, const T* VX, const T* VY, const T* VZ,
                             Buckets<T> out, int min_atoms, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    // (two workgroups per CU in float32, one in float64: a smaller grid costs less when it only skips)
    const int32_t cap = sizeof(T) == 4 ? 1024 : 512;
    const unsigned blocks = static_cast<unsigned>(n_mols < cap ? n_mols : cap);
    aev_fwd_medium_kernel<T, true><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, VX, VY, VZ,
                                                                       out, min_atoms, order, SortedAtoms<T>{});
    return hipGetLastError();
}

template <typename T>
size_t large_scratch_bytes(int64_t n_atoms, int32_t n_mols, bool with_vectors)
{
    return sorted_atoms_bytes<T>(n_atoms, n_mols, with_vectors);
}

// Molecules of more than 256 atoms: the sort into `scratch` (large_scratch_bytes), then the kernel above with the
// centres of a molecule spread over the workgroups of a grid column.
template <typename T>
hipError_t launch_fwd_large(const T* X, const T* Y, const T* Z, const int32_t* A,
                            const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                            const int32_t* SIs, const T* VX, const T* VY, const T* VZ, Buckets<T> out,
                            const int32_t* order, void* scratch, int64_t n_atoms, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const bool jvp = VX != nullptr;
    const SortedAtoms<T> sorted = carve_sorted_atoms<T>(scratch, n_atoms, n_mols, jvp);
    const hipError_t e = launch_large_sort<T>(X, Y, Z, A, MOs, MACs, n_mols, SIs, VX, VY, VZ, nullptr, nullptr, nullptr, order,
                                              sorted, stream);
    if (e != hipSuccess) return e;
    const dim3 grid = large_grid(n_mols);
    if (jvp)
        aev_fwd_medium_kernel<T, true, true><<<grid, dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, VX, VY, VZ, out,
                                                                         kMediumMaxAtoms + 1, order, sorted);
    else
        aev_fwd_medium_kernel<T, false, true><<<grid, dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, nullptr, nullptr,
                                                                          nullptr, out, kMediumMaxAtoms + 1, order, sorted);
    return hipGetLastError();
}

template hipError_t launch_fwd_medium<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<float>, int, const int32_t*, hipStream_t);
template hipError_t launch_fwd_medium<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<double>, int, const int32_t*, hipStream_t);

template hipError_t launch_jvp_medium<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const float*, const float*, const float*, Buckets<float>, int, const int32_t*, hipStream_t);
template hipError_t launch_jvp_medium<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const double*, const double*, const double*, Buckets<double>, int, const int32_t*, hipStream_t);

template size_t large_scratch_bytes<float>(int64_t, int32_t, bool);
template size_t large_scratch_bytes<double>(int64_t, int32_t, bool);
template hipError_t launch_fwd_large<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const float*, const float*, const float*, Buckets<float>, const int32_t*, void*, int64_t, hipStream_t);
template hipError_t launch_fwd_large<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, const double*, const double*, const double*, Buckets<double>, const int32_t*, void*, int64_t, hipStream_t);

}  // namespace khan
