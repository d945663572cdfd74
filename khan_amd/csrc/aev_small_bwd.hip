// AEV backward (dL/dxyz) for molecules of up to 64 atoms, float32: one wavefront per molecule.
//
// Lanes are sorted by atom type and centres are scanned six at a time exactly as in the forward
// kernel, producing per-centre lists of angular partners (unit vector, distance, f_C, f_C').  Then
//   radial   a lane owns one (centre, partner) pair: it reads the 16 upstream values of the partner's
//            type from the centre's row, sums g e (f_C' - 2 eta d f_C) over the shells, and the pull
//            goes to the partner (one group at a time, so targets are distinct) and, summed over the
//            group with DPP moves, to the centre;
//   angular  a lane owns one list entry (centre b, partner j) and walks the other partners of the
//            same centre in round-robin order, k = j+1, j+2, ... (mod m): in every round all lanes of
//            a centre hold distinct j AND distinct k, each unordered pair {j,k} is met exactly once,
//            and all lanes finish together.  A lane computes its triple completely (32 upstream
//            values read straight from the row, three weighted sums formed serially, no cross-lane
//            reduction), keeps the force on j in registers and adds the force on k to a per-centre
//            slot in LDS with a plain read-add-write: targets are distinct by construction, so no
//            atomics are needed (float atomics on LDS cost ~190 cycles per wave instruction here);
//   gather   per centre, the slot of every partner is added to its atom's force, and the centre gets
//            minus the sum (each row's forces add up to zero by translation invariance).
// Finally every lane stores the gradient of its own atom: no global atomics, no pre-zeroed output.
// The derivative is the algebraically reduced form (no acos, no 1/(1+cos) factor); reference:
// gpu_featurizer/kernel_cpu.cpp:217-366.
#include "aev_small_common.h"

namespace khan {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f* global_v4f_ptr;

struct __align__(16) BwdLds {
    float4 atom[64];                     // x, y, z, type (sorted order)
    float4 nbr[kB][kCapA];               // unit vector (centre minus partner)/r, and r
    float4 facc[kB][kCapA];              // force on each partner from its centre's row (xyz, pad)
    float2 nbr_fc[kB][kCapA];            // f_C(r, A_Rc) and its derivative in r
    float force[3][64];                  // dL/dx, dL/dy, dL/dz per sorted atom
    int nM[8];                           // angular partners per centre of the batch
    unsigned char nbr_idx[kB][kCapA];    // sorted lane of the partner
    unsigned char inv[64];               // original atom index -> sorted lane
};

__global__ __launch_bounds__(64 * kWavesPerBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void aev_bwd_small_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<const float> gin, float* __restrict__ gX, float* __restrict__ gY, float* __restrict__ gZ)
{
    __shared__ BwdLds lds_all[kWavesPerBlock];
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int mol = blockIdx.x * kWavesPerBlock + wave;
    if (mol >= n_mols) return;
    const int n = uniform(MACs[mol]);
    const int off = uniform(MOs[mol]);
    if (n <= 0 || n > 64) return;                 // larger molecules belong to the general kernel
    BwdLds& S = lds_all[wave];
    const LaneConsts<float> L = lane_consts<float>(lane);
    const unsigned long long lane_bit = 1ull << lane;
    const unsigned long long lt_mask = lane_bit - 1ull;

    // ------------------------------------------------------------ load, sort lanes by type
    const bool have = lane < n;
    float x = 0.f, y = 0.f, z = 0.f;
    int type = 0, orig = lane;
    unsigned long long rowbits = 0;
    if (have) {
        x = X[off + lane];
        y = Y[off + lane];
        z = Z[off + lane];
        type = fold_type(A[off + lane]);
        rowbits = reinterpret_cast<unsigned long long>(gin.p[type] + static_cast<size_t>(SIs[off + lane]) * kFeats);
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
    S.inv[lane] = static_cast<unsigned char>(dest);
    x = lane_push(dest, x);
    y = lane_push(dest, y);
    z = lane_push(dest, z);
    type = lane_push(dest, type);
    orig = lane_push(dest, orig);
    const int rp_lo = lane_push(dest, static_cast<int>(rowbits & 0xffffffffull));
    const int rp_hi = lane_push(dest, static_cast<int>(rowbits >> 32));
    S.atom[lane] = make_float4(x, y, z, __int_as_float(type));
    S.force[0][lane] = 0.f;
    S.force[1][lane] = 0.f;
    S.force[2][lane] = 0.f;
    auto row_of_lane = [&](int sorted_lane) -> const float* {     // per-lane source index
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(sorted_lane << 2, rp_lo));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(sorted_lane << 2, rp_hi));
        return reinterpret_cast<const float*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };
    auto row_of = [&](int sorted_lane) -> const float* {          // wave-uniform source index
        const unsigned lo = static_cast<unsigned>(lane_read(rp_lo, sorted_lane));
        const unsigned hi = static_cast<unsigned>(lane_read(rp_hi, sorted_lane));
        return reinterpret_cast<const float*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };
    const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
    const int W = 1 << logW, G = 64 >> logW;
    const int grp = lane >> logW, jl = lane & (W - 1);
    const unsigned long long sub_mask = low_bits(W) << ((grp * W) & 63);
    const unsigned long long ltg_mask = lt_mask & sub_mask;
    const float inv_rc_R = 1.0f / kR_Rc_f, inv_rc_A = 1.0f / kA_Rc_f;
    const float kLog2e = 1.44269504088896340736f;
    const float kRadExp = -kR_eta_f * kLog2e;
    const float kAngExp = -kA_eta_f * kLog2e;
    // type of a sorted lane from the type boundaries
    const int tb1 = tbase[1], tb2 = tbase[2], tb3 = tbase[3];
    auto type_of = [&](int sorted_lane) { return (sorted_lane >= tb1) + (sorted_lane >= tb2) + (sorted_lane >= tb3); };
    wave_lds_fence();

    for (int c0 = 0; c0 < n; c0 += kB) {
        const int nb = min(kB, n - c0);
        unsigned overflow = 0;
        for (int q = lane; q < kB * kCapA; q += 64) (&S.facc[0][0])[q] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (lane < 8) S.nM[lane] = 0;
        wave_lds_fence();

        // ------------------------------------------------ scan steps: G centres x W partners
        for (int b0 = 0; b0 < nb; b0 += G) {
            const int b = b0 + grp;
            const int i = c0 + b;
            const bool centre_ok = b < nb;
            const int ci = centre_ok ? i : 0;
            const int cb = centre_ok ? b : 0;
            const float4 ai = S.atom[ci];
            const float4 aj = S.atom[jl];
            const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            const bool inR = valid && (r < kR_Rc_f);
            const bool inA = valid && (r < kA_Rc_f);
            const unsigned long long mA = wave_ballot(inA);
            const int cntA = popc64(mA & sub_mask);
            const bool fits = cntA <= kCapA;
            const float inv = __builtin_amdgcn_rcpf(r);
            if (inA && fits) {
                const int pos = popc64(mA & ltg_mask);
                float fc, dfc;
                cutoff_poly_grad(r * inv_rc_A, inv_rc_A, fc, dfc);
                S.nbr[cb][pos] = make_float4(dx * inv, dy * inv, dz * inv, r);
                S.nbr_fc[cb][pos] = make_float2(fc, dfc);
                S.nbr_idx[cb][pos] = static_cast<unsigned char>(jl);
            }
            if (jl == 0 && centre_ok) S.nM[b] = fits ? cntA : 0;
            {
                const unsigned long long ov = wave_ballot(!fits && jl == 0 && centre_ok);
                for (int g = 0; g < G; ++g)
                    if ((ov >> (g * W)) & 1ull) overflow |= 1u << (b0 + g);
            }

            // ---- radial pairs: this lane's (centre, partner) pair over its 16 shells
            const float* grow = row_of_lane(ci);
            float cfx = 0.f, cfy = 0.f, cfz = 0.f;       // this pair's pull on the centre
            const bool do_rad = inR && fits;              // an overflowing centre is redone as a whole
            if (do_rad) {
                const int tj = __float_as_int(aj.w);
                const global_v4f_ptr gp = (global_v4f_ptr)(grow + tj * kNumRRs);
                const v4f g0 = gp[0], g1 = gp[1], g2 = gp[2], g3 = gp[3];
                const float gr[16] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w,
                                      g2.x, g2.y, g2.z, g2.w, g3.x, g3.y, g3.z, g3.w};
                float fc, dfc;
                cutoff_poly_grad(r * inv_rc_R, inv_rc_R, fc, dfc);
                const float m2eta_fc = -2.0f * kR_eta_f * fc;
                float Gsum = 0.f;
#pragma unroll
                for (int q = 0; q < kNumRRs; ++q) {
                    const float d = r - kR_Rs_f[q];
                    const float e = __builtin_amdgcn_exp2f(kRadExp * d * d);
                    Gsum = fmaf(gr[q] * e, fmaf(m2eta_fc, d, dfc), Gsum);   // g e (f_C' - 2 eta d f_C)
                }
                const float sc = Gsum * inv;           // dE/dr / r, multiplies (x_i - x_j)
                cfx = sc * dx;
                cfy = sc * dy;
                cfz = sc * dz;
            }
            // partner forces: one group per round, so the targets of a round are distinct atoms
            for (int g = 0; g < G; ++g) {
                if (do_rad && grp == g) {
                    S.force[0][jl] -= cfx;
                    S.force[1][jl] -= cfy;
                    S.force[2][jl] -= cfz;
                }
            }
            // the W lanes of a group share their centre: sum inside the group, its last lane adds
            cfx = group_sum_to_last_lane(cfx, logW);
            cfy = group_sum_to_last_lane(cfy, logW);
            cfz = group_sum_to_last_lane(cfz, logW);
            if (jl == W - 1 && centre_ok) {
                S.force[0][i] += cfx;
                S.force[1][i] += cfy;
                S.force[2][i] += cfz;
            }
        }
        wave_lds_fence();

        // ------------------------------------------------ angular: lane = (centre, partner j), round robin over k
        const int4 m03 = *reinterpret_cast<const int4*>(&S.nM[0]);
        const int4 m47 = *reinterpret_cast<const int4*>(&S.nM[4]);
        const int p1 = m03.x, p2 = p1 + m03.y, p3 = p2 + m03.z, p4 = p3 + m03.w, p5 = p4 + m47.x;
        const int total = uniform(p5 + m47.y);
        for (int pass0 = 0; pass0 < total; pass0 += 64) {
            const int slot = pass0 + lane;
            const bool live = slot < total;
            const int b = (slot >= p1) + (slot >= p2) + (slot >= p3) + (slot >= p4) + (slot >= p5);
            const int bs = live ? b : 0;
            const int pb = bs == 0 ? 0 : bs == 1 ? p1 : bs == 2 ? p2 : bs == 3 ? p3 : bs == 4 ? p4 : p5;
            const int m = bs == 0 ? m03.x : bs == 1 ? m03.y : bs == 2 ? m03.z : bs == 3 ? m03.w : bs == 4 ? m47.x : m47.y;
            const int e = live ? slot - pb : 0;
            // rounds: d = 1 .. (m-1)/2 for every lane; when m is even one more round for the lower half
            const int full = (m - 1) >> 1;
            const int rounds = live ? full + ((((m & 1) == 0) && (e < (m >> 1))) ? 1 : 0) : 0;
            const int max_rounds = wave_max(rounds);
            const float4 vj = S.nbr[bs][e];
            const float2 fj = S.nbr_fc[bs][e];
            const int tj = type_of(S.nbr_idx[bs][e]);
            const float inv_rj = __builtin_amdgcn_rcpf(vj.w);
            const float* grow = row_of_lane(c0 + bs);
            float ajx = 0.f, ajy = 0.f, ajz = 0.f;           // force on j, kept in registers

            for (int d = 1; d <= max_rounds; ++d) {
                const bool act = d <= rounds;
                int k = e + d;
                k -= (k >= m) ? m : 0;
                k = act ? k : 0;
                const float4 vk = S.nbr[bs][k];
                const float2 fk = S.nbr_fc[bs][k];
                const int tk = type_of(S.nbr_idx[bs][k]);
                if (act) {
                    const int pt = pair_block(tj, tk);
                    const global_v4f_ptr gp = (global_v4f_ptr)(grow + kRadial + pt * kAngBlock);
                    v4f g[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) g[t] = gp[t];

                    float c = vj.x * vk.x + vj.y * vk.y + vj.z * vk.z;
                    c = fminf(fmaxf(c, -1.0f), 1.0f);
                    const float cx = vj.y * vk.z - vj.z * vk.y;
                    const float cy = vj.z * vk.x - vj.x * vk.z;
                    const float cz = vj.x * vk.y - vj.y * vk.x;
                    // exactly collinear triples have no finite derivative: keep the result finite
                    const float s = fmaxf(__builtin_amdgcn_sqrtf(cx * cx + cy * cy + cz * cz), 1e-30f);
                    const float c_over_s = c * __builtin_amdgcn_rcpf(s);
                    const float rho = 0.5f * (vj.w + vk.w);
                    float Gs[4], Hs[4];
#pragma unroll
                    for (int sidx = 0; sidx < 4; ++sidx) {
                        const float dd = rho - kA_Rs_f[sidx];
                        Gs[sidx] = __builtin_amdgcn_exp2f(kAngExp * dd * dd);
                        Hs[sidx] = Gs[sidx] * (-2.0f * kA_eta_f * dd);          // dG/drho
                    }
                    float W0 = 0.f, Wc = 0.f, Wr = 0.f;
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const float ct = static_cast<float>(kCosTheta[t]), st = static_cast<float>(kSinTheta[t]);
                        const float bs1 = fmaf(s, st, fmaf(c, ct, 1.0f));       // 1 + cos(theta - theta_t)
                        const float b2 = bs1 * bs1, b4 = b2 * b2;
                        const float Am1 = b4 * b2 * bs1;                         // ^7
                        const float At = Am1 * bs1;                              // ^8
                        const float dAt = 8.0f * Am1 * fmaf(-c_over_s, st, ct);  // d/dcos
                        const float ut = g[t].x * Gs[0] + g[t].y * Gs[1] + g[t].z * Gs[2] + g[t].w * Gs[3];
                        const float vt = g[t].x * Hs[0] + g[t].y * Hs[1] + g[t].z * Hs[2] + g[t].w * Hs[3];
                        W0 = fmaf(At, ut, W0);
                        Wc = fmaf(dAt, ut, Wc);
                        Wr = fmaf(At, vt, Wr);
                    }
                    const float two_pow = 0.0078125f;
                    const float P = two_pow * fj.x * fk.x;
                    const float Fj = fmaf(P * 0.5f, Wr, two_pow * W0 * fj.y * fk.x);    // dE/dr_ij
                    const float Fk = fmaf(P * 0.5f, Wr, two_pow * W0 * fj.x * fk.y);    // dE/dr_ik
                    const float Fc = P * Wc;                                            // dE/dcos
                    const float ij = Fc * inv_rj, ik = Fc * __builtin_amdgcn_rcpf(vk.w);
                    ajx -= fmaf(Fj, vj.x, ij * (vk.x - c * vj.x));
                    ajy -= fmaf(Fj, vj.y, ij * (vk.y - c * vj.y));
                    ajz -= fmaf(Fj, vj.z, ij * (vk.z - c * vj.z));
                    // force on k: in a round every lane of a centre holds a different k
                    float4 fk_acc = S.facc[bs][k];
                    fk_acc.x -= fmaf(Fk, vk.x, ik * (vj.x - c * vk.x));
                    fk_acc.y -= fmaf(Fk, vk.y, ik * (vj.y - c * vk.y));
                    fk_acc.z -= fmaf(Fk, vk.z, ik * (vj.z - c * vk.z));
                    S.facc[bs][k] = fk_acc;
                }
                wave_lds_fence();
            }
            if (live) {
                float4 f = S.facc[bs][e];
                f.x += ajx;
                f.y += ajy;
                f.z += ajz;
                S.facc[bs][e] = f;
            }
            wave_lds_fence();
        }

        // ------------------------------------------------ gather: partners get their slot, the centre minus the sum
        for (int b = 0; b < nb; ++b) {
            const int m = b == 0 ? m03.x : b == 1 ? m03.y : b == 2 ? m03.z : b == 3 ? m03.w : b == 4 ? m47.x : m47.y;
            const int mu = uniform(m);
            if (mu == 0) continue;
            float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
            if (lane < mu) {
                f = S.facc[b][lane];
                const int atom = S.nbr_idx[b][lane];
                S.force[0][atom] += f.x;
                S.force[1][atom] += f.y;
                S.force[2][atom] += f.z;
            }
            const float sx = group_sum_to_last_lane(f.x, 6);
            const float sy = group_sum_to_last_lane(f.y, 6);
            const float sz = group_sum_to_last_lane(f.z, 6);
            if (lane == 63) {
                S.force[0][c0 + b] -= sx;
                S.force[1][c0 + b] -= sy;
                S.force[2][c0 + b] -= sz;
            }
            wave_lds_fence();
        }

        // ------------------------------------------------ centres whose list overflowed
        if (overflow) {
            for (int b = 0; b < nb; ++b) {
                if (overflow & (1u << b)) {
                    const int i_orig = lane_read(orig, c0 + b);
                    bwd_center_generic<float>(L, lane, X, Y, Z, A, off, n, i_orig,
                                              reinterpret_cast<float*>(S.nbr), row_of(c0 + b),
                                              [&](int atom, float fx, float fy, float fz) {
                                                  const int sl = S.inv[atom];
                                                  atomicAdd(&S.force[0][sl], fx);
                                                  atomicAdd(&S.force[1][sl], fy);
                                                  atomicAdd(&S.force[2][sl], fz);
                                              });
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

hipError_t launch_bwd_small_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                const int32_t* SIs, Buckets<const float> g, float* gX, float* gY,
                                float* gZ, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kWavesPerBlock - 1u) / kWavesPerBlock;
    aev_bwd_small_kernel<<<dim3(blocks), dim3(64 * kWavesPerBlock), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ);
    return hipGetLastError();
}

}  // namespace khan
