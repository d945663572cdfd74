// AEV backward (dL/dxyz) for molecules of up to 64 atoms, float32: one wavefront per molecule.
//
// Lanes are sorted by atom type as in the forward kernel.  A first sweep counts the angular partners
// of every atom; centres are then taken in order of decreasing count, in batches of up to six whose
// partner lists together fill at most the 64 lanes.  Per batch:
//   stage    the 320 angular upstream values of each centre's row are fetched with full-line loads
//            (issued before the scan, so their latency is covered) and laid out in LDS by type pair;
//   scan     64 (centre, partner) pairs per step; angular partners (unit vector, distance, f_C, f_C')
//            go to one pooled list, centre after centre;
//   radial   a lane owns one (centre, partner) pair: it reads the 16 upstream values of the partner's
//            type from the centre's row, sums g e (f_C' - 2 eta d f_C) over the shells, and the pull
//            goes to the partner (one group at a time, so targets are distinct) and, summed over the
//            group with DPP moves, to the centre;
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
#include "aev_small_common.h"

namespace khan {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f* global_v4f_ptr;

constexpr int kBlockStride = 36;   // floats between staged 32-float blocks: rotates the LDS banks

struct __align__(16) BwdLds {
    float4 atom[64];                              // x, y, z, type (sorted order)
    float4 nbr[64];                               // pooled lists: unit vector (centre minus partner)/r, and r
    float4 facc[64];                              // force on each list entry from its centre's row
    float2 nbr_fc[64];                            // f_C(r, A_Rc) and its derivative in r
    float gst[kB * kNumPairBlocks * kBlockStride];   // staged upstream blocks [centre][type pair][32]
    float force[3][64];                           // dL/dx, dL/dy, dL/dz per sorted atom
    int nM[8];                                    // angular partners per centre of the batch
    unsigned char nbr_idx[64];                    // sorted lane of the partner
    unsigned char inv[64];                        // original atom index -> sorted lane
};

__device__ __forceinline__ int sel6(int b, int v0, int v1, int v2, int v3, int v4, int v5)
{
    return b == 0 ? v0 : b == 1 ? v1 : b == 2 ? v2 : b == 3 ? v3 : b == 4 ? v4 : v5;
}

__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3, 3))) void aev_bwd_small_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<const float> gin, float* __restrict__ gX, float* __restrict__ gY, float* __restrict__ gZ)
{
    __shared__ BwdLds S;
    const int lane = threadIdx.x;
    const int mol = blockIdx.x;
    if (mol >= n_mols) return;
    const int n = uniform(MACs[mol]);
    const int off = uniform(MOs[mol]);
    if (n <= 0 || n > 64) return;                 // larger molecules belong to the general kernel
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
    const float4 aj = S.atom[jl];      // the partner this lane tests in every scan step

    // ------------------------------------------------------------ order of the centres
    // Angular partner count of every atom, then centres in order of decreasing count: a batch of
    // centres shares the lanes of the round-robin walk and runs as long as its busiest centre, so
    // centres with similar counts go together and a batch is cut where its lists fill the 64 lanes.
    int cord, m_at;     // lane p: sorted lane of the centre at position p, and its partner count
    {
        int m_mine = 0;
        for (int s0 = 0; s0 < n; s0 += G) {
            const int i = s0 + grp;
            const float4 ai = S.atom[min(i, 63)];
            const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool inA = (i < n) && (jl < n) && (jl != i) && (r < kA_Rc_f);
            const int cnt = popc64(wave_ballot(inA) & sub_mask);          // in every lane of the group
            const int got = __builtin_amdgcn_ds_bpermute((((lane - s0) << logW) & 63) << 2, cnt);
            if (lane >= s0 && lane < s0 + G) m_mine = got;
        }
        const int key = have ? ((m_mine << 6) | (63 - lane)) : -1;
        int rank = 0;
        for (int l = 0; l < n; ++l) rank += (lane_read(key, l) > key) ? 1 : 0;
        if (!have) rank = lane;
        cord = lane_push(rank, lane);
        m_at = lane_push(rank, m_mine);
    }

    for (int c0 = 0, nb = 0; c0 < n; c0 += nb) {
        // centres of this batch: up to kB, lists fitting the 64 lanes; pf[b] = first list slot of centre b
        int pf[kB + 1];
        {
            bool open = true;
            int tot = 0;
            nb = 0;
            pf[0] = 0;
#pragma unroll
            for (int k = 0; k < kB; ++k) {
                int m = 0;
                if (open && c0 + k < n) {
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
        v4f st0[kB], st1[kB];
#pragma unroll
        for (int b = 0; b < kB; ++b) {
            st0[b] = v4f{0.f, 0.f, 0.f, 0.f};
            st1[b] = v4f{0.f, 0.f, 0.f, 0.f};
            if (b < nb) {
                const global_v4f_ptr rowp = (global_v4f_ptr)(row_of(lane_read(cord, min(c0 + b, 63))) + kRadial);
                st0[b] = rowp[lane];
                if (lane < 16) st1[b] = rowp[64 + lane];
            }
        }
        S.facc[lane] = make_float4(0.f, 0.f, 0.f, 0.f);
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
            const float4 ai = S.atom[i];
            const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            const bool inR = valid && (r < kR_Rc_f);
            const bool inA = valid && (r < kA_Rc_f);
            const unsigned long long mA = wave_ballot(inA);
            const int cntA = popc64(mA & sub_mask);
            const bool fits = cntA == room;       // the list has the length the first sweep counted
            const float inv = __builtin_amdgcn_rcpf(r);
            if (inA && fits) {
                const int pos = base + popc64(mA & ltg_mask);
                float fc, dfc;
                cutoff_poly_grad(r * inv_rc_A, inv_rc_A, fc, dfc);
                S.nbr[pos] = make_float4(dx * inv, dy * inv, dz * inv, r);
                S.nbr_fc[pos] = make_float2(fc, dfc);
                S.nbr_idx[pos] = static_cast<unsigned char>(jl);
            }
            if (jl == 0 && centre_ok) S.nM[b] = fits ? cntA : 0;
            {
                const unsigned long long ov = wave_ballot(!fits && jl == 0 && centre_ok);
                for (int g = 0; g < G; ++g)
                    if ((ov >> (g * W)) & 1ull) overflow |= 1u << (b0 + g);
            }

            // ---- radial pairs: this lane's (centre, partner) pair over its 16 shells
            const float* grow = row_of_lane(i);
            float cfx = 0.f, cfy = 0.f, cfz = 0.f;       // this pair's pull on the centre
            const bool do_rad = inR && fits;              // a centre that does not fit is redone as a whole
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

        // ---- the fetched upstream blocks go to LDS: chunk c of a row = block c/8, part c%8
#pragma unroll
        for (int b = 0; b < kB; ++b) {
            if (b < nb) {
                float* blk = &S.gst[b * kNumPairBlocks * kBlockStride];
                *reinterpret_cast<v4f*>(blk + (lane >> 3) * kBlockStride + (lane & 7) * 4) = st0[b];
                if (lane < 16) *reinterpret_cast<v4f*>(blk + (8 + (lane >> 3)) * kBlockStride + (lane & 7) * 4) = st1[b];
            }
        }
        wave_lds_fence();

        // ------------------------------------------------ angular: lane = list entry (centre, partner j)
        {
            const int4 m03 = *reinterpret_cast<const int4*>(&S.nM[0]);
            const int4 m47 = *reinterpret_cast<const int4*>(&S.nM[4]);
            const int b = (lane >= pf[1]) + (lane >= pf[2]) + (lane >= pf[3]) + (lane >= pf[4]) + (lane >= pf[5]);
            const int bs = lane < total ? b : 0;
            const int pb = sel6(bs, pf[0], pf[1], pf[2], pf[3], pf[4], pf[5]);
            const int m = sel6(bs, m03.x, m03.y, m03.z, m03.w, m47.x, m47.y);   // 0 for a centre that did not fit
            const bool live = (lane < total) && (m > 0);
            const int e = live ? lane - pb : 0;
            // rounds: d = 1 .. (m-1)/2 for every lane; when m is even one more round for the lower half
            const int full = (m - 1) >> 1;
            const int rounds = live ? full + ((((m & 1) == 0) && (e < (m >> 1))) ? 1 : 0) : 0;
            const int max_rounds = wave_max(rounds);
            const int self = live ? lane : 0;
            const float4 vj = S.nbr[self];
            const float2 fj = S.nbr_fc[self];
            const int tj = type_of(S.nbr_idx[self]);
            const float inv_rj = __builtin_amdgcn_rcpf(vj.w);
            const float* gbase = &S.gst[bs * kNumPairBlocks * kBlockStride];
            float ajx = 0.f, ajy = 0.f, ajz = 0.f;           // force on j, kept in registers

            for (int d = 1; d <= max_rounds; ++d) {
                const bool act = d <= rounds;
                int k = e + d;
                k -= (k >= m) ? m : 0;
                const int ks = act ? pb + k : 0;
                const float4 vk = S.nbr[ks];
                const float2 fk = S.nbr_fc[ks];
                const int tk = type_of(S.nbr_idx[ks]);
                if (act) {
                    const v4f* gp = reinterpret_cast<const v4f*>(gbase + pair_block(tj, tk) * kBlockStride);
                    v4f g[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) g[t] = gp[t];

                    float c = vj.x * vk.x + vj.y * vk.y + vj.z * vk.z;
                    c = fminf(fmaxf(c, -1.0f), 1.0f);
                    const float cx = vj.y * vk.z - vj.z * vk.y;
                    const float cy = vj.z * vk.x - vj.x * vk.z;
                    const float cz = vj.x * vk.y - vj.y * vk.x;
                    // cot(theta) = c/s has no limit for collinear triples (the angle has a cusp there, the
                    // reference returns NaN): c s / (s^2 + 1e-12) equals c/s to 1e-7 relative from 0.2 degrees
                    // off the line and goes to zero on it
                    const float s2 = cx * cx + cy * cy + cz * cz;
                    const float s = __builtin_amdgcn_sqrtf(s2);
                    const float c_over_s = c * s * __builtin_amdgcn_rcpf(s2 + 1e-12f);
                    const float rho = 0.5f * (vj.w + vk.w);
                    float Gs[4], dds[4];
#pragma unroll
                    for (int sidx = 0; sidx < 4; ++sidx) {
                        dds[sidx] = rho - kA_Rs_f[sidx];
                        Gs[sidx] = __builtin_amdgcn_exp2f(kAngExp * dds[sidx] * dds[sidx]);
                    }
                    // X_s = sum_t g_ts A_t and Y_s = sum_t g_ts dA_t/dcos (without its factor 8)
                    float Xs[4] = {0.f, 0.f, 0.f, 0.f}, Ys[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const float ct = static_cast<float>(kCosTheta[t]), st = static_cast<float>(kSinTheta[t]);
                        const float bs1 = fmaf(s, st, fmaf(c, ct, 1.0f));       // 1 + cos(theta - theta_t)
                        const float b2 = bs1 * bs1, b4 = b2 * b2;
                        const float Am1 = b4 * b2 * bs1;                         // ^7
                        const float At = Am1 * bs1;                              // ^8
                        const float dAt = Am1 * fmaf(-c_over_s, st, ct);         // (d/dcos) / 8
                        Xs[0] = fmaf(g[t].x, At, Xs[0]);
                        Xs[1] = fmaf(g[t].y, At, Xs[1]);
                        Xs[2] = fmaf(g[t].z, At, Xs[2]);
                        Xs[3] = fmaf(g[t].w, At, Xs[3]);
                        Ys[0] = fmaf(g[t].x, dAt, Ys[0]);
                        Ys[1] = fmaf(g[t].y, dAt, Ys[1]);
                        Ys[2] = fmaf(g[t].z, dAt, Ys[2]);
                        Ys[3] = fmaf(g[t].w, dAt, Ys[3]);
                    }
                    // W0 = sum G_s X_s, Wc = 8 sum G_s Y_s, Wr = sum (dG_s/drho) X_s with dG/drho = -2 eta dd G
                    const float gx0 = Gs[0] * Xs[0], gx1 = Gs[1] * Xs[1], gx2 = Gs[2] * Xs[2], gx3 = Gs[3] * Xs[3];
                    const float W0 = (gx0 + gx1) + (gx2 + gx3);
                    const float Wc = 8.0f * fmaf(Gs[0], Ys[0], fmaf(Gs[1], Ys[1], fmaf(Gs[2], Ys[2], Gs[3] * Ys[3])));
                    const float Wr = (-2.0f * kA_eta_f) * fmaf(dds[0], gx0, fmaf(dds[1], gx1, fmaf(dds[2], gx2, dds[3] * gx3)));
                    const float two_pow = 0.0078125f;
                    const float P = two_pow * fj.x * fk.x;
                    const float Fj = fmaf(P * 0.5f, Wr, two_pow * W0 * fj.y * fk.x);    // dE/dr_ij
                    const float Fk = fmaf(P * 0.5f, Wr, two_pow * W0 * fj.x * fk.y);    // dE/dr_ik
                    const float Fc = P * Wc;                                            // dE/dcos
                    const float ij = Fc * inv_rj, ik = Fc * __builtin_amdgcn_rcpf(vk.w);
                    // force on j = -[Fj u_j + ij (u_k - c u_j)]; the bracket's second part is formed first, it
                    // is small near the line where ij is large
                    ajx = fmaf(-Fj, vj.x, fmaf(-ij, fmaf(-c, vj.x, vk.x), ajx));
                    ajy = fmaf(-Fj, vj.y, fmaf(-ij, fmaf(-c, vj.y, vk.y), ajy));
                    ajz = fmaf(-Fj, vj.z, fmaf(-ij, fmaf(-c, vj.z, vk.z), ajz));
                    // force on k: in a round every lane of a centre holds a different k
                    float4 fk_acc = S.facc[ks];
                    fk_acc.x = fmaf(-Fk, vk.x, fmaf(-ik, fmaf(-c, vk.x, vj.x), fk_acc.x));
                    fk_acc.y = fmaf(-Fk, vk.y, fmaf(-ik, fmaf(-c, vk.y, vj.y), fk_acc.y));
                    fk_acc.z = fmaf(-Fk, vk.z, fmaf(-ik, fmaf(-c, vk.z, vj.z), fk_acc.z));
                    S.facc[ks] = fk_acc;
                }
                wave_lds_fence();
            }

            // -------------------------------------------- gather: partners get their slot, the centre minus the sum
            float4 f = S.facc[self];
            f.x = live ? f.x + ajx : 0.f;
            f.y = live ? f.y + ajy : 0.f;
            f.z = live ? f.z + ajz : 0.f;
            const int atom = S.nbr_idx[self];
            for (int bb = 0; bb < nb; ++bb) {
                if (uniform(pf[bb + 1] - pf[bb]) == 0) continue;
                const bool mine = live && (bs == bb);
                if (mine) {
                    S.force[0][atom] += f.x;
                    S.force[1][atom] += f.y;
                    S.force[2][atom] += f.z;
                }
                const float sx = group_sum_to_last_lane(mine ? f.x : 0.f, 6);
                const float sy = group_sum_to_last_lane(mine ? f.y : 0.f, 6);
                const float sz = group_sum_to_last_lane(mine ? f.z : 0.f, 6);
                if (lane == 63) {
                    const int i_b = lane_read(cord, min(c0 + bb, 63));
                    S.force[0][i_b] -= sx;
                    S.force[1][i_b] -= sy;
                    S.force[2][i_b] -= sz;
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
                    bwd_center_generic<float>(L, lane, X, Y, Z, A, off, n, i_orig, S.gst, row_of(i_b),
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
    aev_bwd_small_kernel<<<dim3(static_cast<unsigned>(n_mols)), dim3(64), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ);
    return hipGetLastError();
}

}  // namespace khan
