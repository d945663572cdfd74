// AEV forward for molecules of 65 to 256 atoms (float32): one workgroup of four wavefronts per molecule.
//
// The workgroup sorts the molecule's atoms by type into LDS once (256-way counting sort with per-wave
// ballots).  Each wavefront then takes batches of six centres and runs the same pipeline as the
// one-wavefront-per-molecule kernel on them:
//   scan     a centre is tested against the sorted atoms 64 at a time; partners inside the radial
//            cutoff are appended to a (r, f_C) list, partners inside the angular cutoff to the centre's
//            list of unit vectors.  Chunks are consecutive ranges of the sorted order, so both lists
//            stay sorted by type.
//   radial   lanes = (slot of 4) x (shell): a centre's list is walked type by type, sixteen entries per
//            trip, and 16 finished floats per type go straight to the row.
//   angular  segment table, triple-per-lane factors and the (theta_t, Rs_s) accumulation of the shared
//            batch routine.
// Rows are written once, without atomics.  A centre with more than 32 angular or 64 radial partners is
// redone by the general per-centre routine.  Semantics: gpu_featurizer/kernel_cpu.cpp:406-537.
#include "aev_fwd_batch.h"

namespace khan {

namespace {

constexpr int kMedMin = kSmallPreferredMax + 1;   // smaller molecules run one wavefront each
constexpr int kRadCap = 64;                   // radial partners kept per centre
constexpr int kMedRadTrip = 1;                // list entries a lane takes per trip of the radial walk (four slots: 4 entries per trip)

struct __align__(16) MedShared {
    float4 atom[kMediumMaxAtoms];          // x, y, z, type (sorted order)
    unsigned row_lo[kMediumMaxAtoms];      // address of the atom's output row
    unsigned row_hi[kMediumMaxAtoms];
    unsigned short orig[kMediumMaxAtoms];  // sorted position -> index inside the molecule
    int wcount[4][4];                      // atoms of each type held by each wavefront before the sort
};

__global__ __launch_bounds__(256) void aev_fwd_medium_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<float> out, const int32_t* __restrict__ order)
{
    __shared__ MedShared M;
    __shared__ FwdWaveLds<float> lds_wave[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    FwdWaveLds<float>& S = lds_wave[wave];
    const LaneConsts<float> L = lane_consts<float>(lane);
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    const float inv_rc_R = 1.0f / kR_Rc_f, inv_rc_A = 1.0f / kA_Rc_f;
    const float kRadExp = -kR_eta_f * 1.44269504088896340736f;   // exp(-eta d^2) = exp2(kRadExp d^2)
    const int rslot = lane >> 4;                                 // radial walk: entry slot of this 16-lane group

    fwd_lds_init(S, lane);
    __shared__ unsigned long long want[4];
    for_each_molecule_in_range(MACs, n_mols, kMedMin, kMediumMaxAtoms, want, order, order ? order + n_mols : nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);

        // ------------------------------------------------------------ load, sort by type into LDS
        const bool have = tid < n;
        float x = 0.f, y = 0.f, z = 0.f;
        int type = 0;
        unsigned long long rowbits = 0;
        if (have) {
            x = X[off + tid];
            y = Y[off + tid];
            z = Z[off + tid];
            type = fold_type(A[off + tid]);
            rowbits = reinterpret_cast<unsigned long long>(out.p[type] + static_cast<size_t>(SIs[off + tid]) * kFeats);
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
            M.atom[dest] = make_float4(x, y, z, __int_as_float(type));
            M.row_lo[dest] = static_cast<unsigned>(rowbits & 0xffffffffull);
            M.row_hi[dest] = static_cast<unsigned>(rowbits >> 32);
            M.orig[dest] = static_cast<unsigned short>(tid);
        }
        __syncthreads();
        auto row_of = [&](int sorted_idx) -> float* {            // wave-uniform index
            const unsigned lo = static_cast<unsigned>(uniform(static_cast<int>(M.row_lo[sorted_idx])));
            const unsigned hi = static_cast<unsigned>(uniform(static_cast<int>(M.row_hi[sorted_idx])));
            return reinterpret_cast<float*>((static_cast<unsigned long long>(hi) << 32) | lo);
        };

        // ------------------------------------------------------------ batches of six centres per wavefront
        for (int c0 = wave * kFB; c0 < n; c0 += 4 * kFB) {
            const int nb = min(kFB, n - c0);
            unsigned overflow = 0;

            for (int b = 0; b < nb; ++b) {
                const int i = c0 + b;
                const float4 ai = M.atom[i];
                int posR = 0, posA = 0;                 // list lengths so far (wave-uniform)
                int cR[4] = {0, 0, 0, 0}, cA[4] = {0, 0, 0, 0};
                for (int jc = 0; jc < n; jc += 64) {
                    const int j = jc + lane;
                    const float4 aj = M.atom[min(j, kMediumMaxAtoms - 1)];
                    const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
                    const float r = sqrtf(dx * dx + dy * dy + dz * dz);
                    const bool valid = (j < n) && (j != i);
                    const bool inR = valid && (r < kR_Rc_f);
                    const bool inA = valid && (r < kA_Rc_f);
                    const unsigned long long mR = wave_ballot(inR), mA = wave_ballot(inA);
                    const int tj = __float_as_int(aj.w);
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const unsigned long long ta = wave_ballot(tj == a);
                        cR[a] += popc64(mR & ta);
                        cA[a] += popc64(mA & ta);
                    }
                    if (inR) {
                        const int p = posR + popc64(mR & lt_mask);
                        if (p < kRadCap) S.rad[p] = make_float2(r, cutoff_poly(r * inv_rc_R));
                    }
                    if (inA) {
                        const int p = posA + popc64(mA & lt_mask);
                        if (p < kCapA) {
                            const float inv = __builtin_amdgcn_rcpf(r);
                            S.nbr[b][p] = make_float4(dx * inv, dy * inv, dz * inv, r);
                            S.nbr_fc[b][p] = cutoff_poly(r * inv_rc_A);
                        }
                    }
                    posR += popc64(mR);
                    posA += popc64(mA);
                }
                const bool fits = (posR <= kRadCap) && (posA <= kCapA);
                if (!fits) overflow |= 1u << b;
                if (lane < 4) S.nA[b][lane] = fits ? sel4(lane, cA[0], cA[1], cA[2], cA[3]) : 0;
                wave_lds_fence();

                // ---- radial features of this centre: lanes = (slot of 4) x (shell)
                if (fits) {
                    float* row = row_of(i);
                    int obase = 0;
#pragma unroll
                    for (int a = 0; a < 4; ++a) {
                        const int cnt_a = cR[a];
                        float acc_r = 0.f;
                        for (int q0 = 0; q0 < cnt_a; q0 += 4 * kMedRadTrip) {
                            float2 e[kMedRadTrip];
#pragma unroll
                            for (int u = 0; u < kMedRadTrip; ++u) e[u] = S.rad[min(obase + q0 + u * 4 + rslot, kRadCap - 1)];
#pragma unroll
                            for (int u = 0; u < kMedRadTrip; ++u) {
                                const float dd = e[u].x - L.rrs;
                                const float v = __builtin_amdgcn_exp2f(kRadExp * dd * dd) * e[u].y;
                                acc_r += (q0 + u * 4 + rslot < cnt_a) ? v : 0.f;   // entries of other types: select
                            }
                        }
                        acc_r += __shfl_xor(acc_r, 16, 64);
                        acc_r += __shfl_xor(acc_r, 32, 64);
                        if (rslot == 0) store_global(row + a * kNumRRs + (lane & 15), acc_r);
                        obase += cnt_a;
                    }
                }
                wave_lds_fence();
            }

            // ------------------------------------------------ segment table, phases 1 and 2, zero fill
            fwd_angular_batch<float, false>(S, L, lane, nb, [&](int b) -> unsigned long long {
                const int idx = min(c0 + b, kMediumMaxAtoms - 1);
                return (static_cast<unsigned long long>(M.row_hi[idx]) << 32) | M.row_lo[idx];
            });

            // ------------------------------------------------ centres whose lists overflowed
            if (overflow) {
                __threadfence();
                for (int b = 0; b < nb; ++b) {
                    if (overflow & (1u << b)) {
                        const int i_orig = uniform(static_cast<int>(M.orig[c0 + b]));
                        fwd_center_generic<float>(L, lane, X, Y, Z, A, off, n, i_orig,
                                                  reinterpret_cast<float*>(S.rec), row_of(c0 + b));
                    }
                }
                wave_lds_fence();
            }
        }
        __syncthreads();      // the next molecule reuses the sorted arrays
    });
}

}  // namespace

hipError_t launch_fwd_medium_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                 const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                 const int32_t* SIs, Buckets<float> out, const int32_t* order, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    // workgroups walk the molecules with the grid's stride and skip those of other sizes
    const unsigned blocks = static_cast<unsigned>(n_mols < 4096 ? n_mols : 4096);
    aev_fwd_medium_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, out, order);
    return hipGetLastError();
}

}  // namespace khan
