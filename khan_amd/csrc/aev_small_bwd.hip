// AEV backward (dL/dxyz) for molecules of up to 64 atoms, float32: one wavefront per molecule.
//
// Same skeleton as the small-molecule forward kernel (lanes sorted by type, six centres per batch,
// scan steps of G centres x W partners, type-sorted neighbour lists in LDS, triples enumerated in
// (centre, type-pair) order and dealt one per lane), but here a lane owns its triple completely:
// it recomputes the geometry, reads the 32 upstream values g[type pair][theta_t][Rs_s] of its centre
// straight from the upstream row (lanes of one segment read the same 128 bytes, served by the
// vector L1), forms the three weighted sums
//     W0 = sum g A_t G_s,   Wc = sum g dA_t/dcos G_s,   Wr = sum g A_t dG_s/drho
// serially over the 32 slots -- no cross-lane reduction -- and adds the forces on i, j and k into
// a per-molecule force array in LDS.  Radial pairs are handled the same way in the scan step, one
// (centre, partner) pair per lane over its 16 shells.  When the molecule is finished each lane
// stores the gradient of its own atom: no global atomics, no pre-zeroed output.
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
    float2 nbr_fc[kB][kCapA];            // f_C(r, A_Rc) and its derivative in r
    float force[3][64];                  // dL/dx, dL/dy, dL/dz per sorted atom
    SegDesc seg[64];
    unsigned bits[kBitWords];
    int nA[kB][4];
    unsigned char nbr_idx[kB][kCapA];    // sorted lane of the partner
    unsigned char inv[64];               // original atom index -> sorted lane
};

__global__ __launch_bounds__(256) void aev_bwd_small_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<const float> gin, float* __restrict__ gX, float* __restrict__ gY, float* __restrict__ gZ)
{
    __shared__ BwdLds lds_all[4];
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int mol = blockIdx.x * 4 + wave;
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
    unsigned long long smask[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) smask[a] = (tcount[a] == 0) ? 0ull : (low_bits(tcount[a]) << tbase[a]);

    const int logW = n <= 16 ? 4 : n <= 32 ? 5 : 6;
    const int W = 1 << logW, G = 64 >> logW;
    const int grp = lane >> logW, jl = lane & (W - 1);
    const unsigned long long sub_mask = low_bits(W) << ((grp * W) & 63);
    const unsigned long long ltg_mask = lt_mask & sub_mask;
    const int cl_g = (lane >> 2) & 3, cl_a = lane & 3;
    const bool cl_on = (lane < 16) && (cl_g < G);
    const unsigned long long cl_sub = cl_on ? (low_bits(W) << ((cl_g * W) & 63)) : 0ull;
    const unsigned long long cl_mask =
        cl_on ? ((cl_a == 0 ? smask[0] : cl_a == 1 ? smask[1] : cl_a == 2 ? smask[2] : smask[3]) << ((cl_g * W) & 63)) : 0ull;

    const int seg_b = lane / kNumPairBlocks, seg_pt = lane - seg_b * kNumPairBlocks;
    const int seg_a = seg_pt < 4 ? 0 : seg_pt < 7 ? 1 : seg_pt < 9 ? 2 : 3;
    const int seg_bt = seg_pt < 4 ? seg_pt : seg_pt < 7 ? seg_pt - 3 : seg_pt < 9 ? seg_pt - 5 : 3;

    const float inv_rc_R = 1.0f / kR_Rc_f, inv_rc_A = 1.0f / kA_Rc_f;
    const float kLog2e = 1.44269504088896340736f;
    const float kRadExp = -kR_eta_f * kLog2e;
    const float kAngExp = -kA_eta_f * kLog2e;
    wave_lds_fence();

    for (int c0 = 0; c0 < n; c0 += kB) {
        const int nb = min(kB, n - c0);
        unsigned overflow = 0;

        // ------------------------------------------------ scan steps: G centres x W partners
        for (int b0 = 0; b0 < nb; b0 += G) {
            const int b = b0 + grp;
            const int i = c0 + b;
            const bool centre_ok = b < nb;
            const int ci = centre_ok ? i : 0;
            const float4 ai = S.atom[ci];
            const float4 aj = S.atom[jl];
            const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            const bool inR = valid && (r < kR_Rc_f);
            const bool inA = valid && (r < kA_Rc_f);
            const unsigned long long mA = wave_ballot(inA);
            const bool fits = popc64(mA & sub_mask) <= kCapA;
            const float inv = __builtin_amdgcn_rcpf(r);
            if (inA && fits) {
                const int pos = popc64(mA & ltg_mask);
                float fc, dfc;
                cutoff_poly_grad(r * inv_rc_A, inv_rc_A, fc, dfc);
                S.nbr[ci - c0][pos] = make_float4(dx * inv, dy * inv, dz * inv, r);
                S.nbr_fc[ci - c0][pos] = make_float2(fc, dfc);
                S.nbr_idx[ci - c0][pos] = static_cast<unsigned char>(jl);
            }
            {
                const unsigned long long ov = wave_ballot(!fits && jl == 0 && centre_ok);
                for (int g = 0; g < G; ++g)
                    if ((ov >> (g * W)) & 1ull) overflow |= 1u << (b0 + g);
            }
            if (cl_on) {
                const int cb = b0 + cl_g;
                if (cb < nb) S.nA[cb][cl_a] = (popc64(mA & cl_sub) <= kCapA) ? popc64(mA & cl_mask) : 0;
            }

            // ---- radial pairs: this lane's (centre, partner) pair over its 16 shells
            const float* grow = row_of_lane(ci);
            float cfx = 0.f, cfy = 0.f, cfz = 0.f;       // this pair's pull on the centre
            if (inR && fits) {      // an overflowing centre is redone as a whole by the general routine
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
                atomicAdd(&S.force[0][jl], -cfx);
                atomicAdd(&S.force[1][jl], -cfy);
                atomicAdd(&S.force[2][jl], -cfz);
            }
            // the W lanes of a group share their centre: sum inside the group, one lane adds
            cfx = group_sum_to_last_lane(cfx, logW);
            cfy = group_sum_to_last_lane(cfy, logW);
            cfz = group_sum_to_last_lane(cfz, logW);
            if (jl == W - 1 && centre_ok) {
                atomicAdd(&S.force[0][i], cfx);
                atomicAdd(&S.force[1][i], cfy);
                atomicAdd(&S.force[2][i], cfz);
            }
        }
        wave_lds_fence();

        // ------------------------------------------------ segment table of the batch
        int cnt = 0, packed = 0;
        float rcp_na = 0.f;
        if (lane < nb * kNumPairBlocks) {
            const int4 nn = *reinterpret_cast<const int4*>(S.nA[seg_b]);
            const int na = sel4(seg_a, nn.x, nn.y, nn.z, nn.w);
            const int nbt = sel4(seg_bt, nn.x, nn.y, nn.z, nn.w);
            const int oa = sel4(seg_a, 0, nn.x, nn.x + nn.y, nn.x + nn.y + nn.z);
            const int ob = sel4(seg_bt, 0, nn.x, nn.x + nn.y, nn.x + nn.y + nn.z);
            const bool same = seg_a == seg_bt;
            cnt = same ? (na * (na - 1)) / 2 : na * nbt;
            packed = seg_b | (oa << 3) | (ob << 9) | (na << 15) | (same ? (1 << 21) : 0) | (seg_pt << 22);
            rcp_na = na > 0 ? __builtin_amdgcn_rcpf(static_cast<float>(na)) : 0.f;
        }
        const int incl = scan_add(cnt);
        const int start = incl - cnt;
        const int total = lane_read(incl, 63);
        const unsigned long long nonempty = wave_ballot(cnt > 0);
        for (int w = lane; w < kBitWords; w += 64) S.bits[w] = 0u;
        wave_lds_fence();
        if (cnt > 0) {
            SegDesc d;
            d.start = start;
            d.cnt = cnt;
            d.packed = packed;
            d.rcp_na = rcp_na;
            S.seg[popc64(nonempty & lt_mask)] = d;
            atomicOr(&S.bits[start >> 5], 1u << (start & 31));
        }
        wave_lds_fence();

        // ------------------------------------------------ triples, one per lane
        int carry = 0;
        for (int base = 0; base < total; base += 64) {
            const unsigned w0 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[base >> 5])));
            const unsigned w1 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[(base >> 5) + 1])));
            const unsigned long long starts = (static_cast<unsigned long long>(w1) << 32) | w0;
            const int ord = carry + popc64(starts & (lt_mask | lane_bit)) - 1;
            carry += popc64(starts);
            const SegDesc d = S.seg[max(ord, 0)];
            const int slot = base + lane;
            const int q = slot - d.start;
            const bool ok = (slot < total) && (q >= 0) && (q < d.cnt);

            int bsel = d.packed & 7;
            const int oa = (d.packed >> 3) & 63, ob = (d.packed >> 9) & 63, na = (d.packed >> 15) & 63;
            const int pt = (d.packed >> 22) & 15;
            int kl, jl2;
            if ((d.packed >> 21) & 1) {
                kl = static_cast<int>((1.0f + __builtin_amdgcn_sqrtf(8.0f * static_cast<float>(q) + 1.0f)) * 0.5f);
                if ((kl * (kl - 1)) / 2 > q) --kl;
                if (((kl + 1) * kl) / 2 <= q) ++kl;
                jl2 = q - (kl * (kl - 1)) / 2;
            } else {
                kl = static_cast<int>((static_cast<float>(q) + 0.5f) * d.rcp_na);
                jl2 = q - kl * na;
            }
            int j = oa + jl2, k = ob + kl;
            if (!ok) {
                j = 0;
                k = 0;
                bsel = 0;
            }
            const float* grow = row_of_lane(c0 + bsel);
            float cix = 0.f, ciy = 0.f, ciz = 0.f;       // this triple's pull on its centre
            if (ok) {
                const global_v4f_ptr gp = (global_v4f_ptr)(grow + kRadial + pt * kAngBlock);
                v4f g[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) g[t] = gp[t];
                const float4 vj = S.nbr[bsel][j], vk = S.nbr[bsel][k];
                const float2 fj = S.nbr_fc[bsel][j], fk = S.nbr_fc[bsel][k];
                const int atom_j = S.nbr_idx[bsel][j], atom_k = S.nbr_idx[bsel][k];

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
                    const float bs = fmaf(s, st, fmaf(c, ct, 1.0f));        // 1 + cos(theta - theta_t)
                    const float b2 = bs * bs, b4 = b2 * b2;
                    const float Am1 = b4 * b2 * bs;                          // ^7
                    const float At = Am1 * bs;                               // ^8
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
                const float ij = Fc * __builtin_amdgcn_rcpf(vj.w), ik = Fc * __builtin_amdgcn_rcpf(vk.w);
                const float vjx = fmaf(Fj, vj.x, ij * (vk.x - c * vj.x));
                const float vjy = fmaf(Fj, vj.y, ij * (vk.y - c * vj.y));
                const float vjz = fmaf(Fj, vj.z, ij * (vk.z - c * vj.z));
                const float vkx = fmaf(Fk, vk.x, ik * (vj.x - c * vk.x));
                const float vky = fmaf(Fk, vk.y, ik * (vj.y - c * vk.y));
                const float vkz = fmaf(Fk, vk.z, ik * (vj.z - c * vk.z));
                cix = vjx + vkx;
                ciy = vjy + vky;
                ciz = vjz + vkz;
                atomicAdd(&S.force[0][atom_j], -vjx);
                atomicAdd(&S.force[1][atom_j], -vjy);
                atomicAdd(&S.force[2][atom_j], -vjz);
                atomicAdd(&S.force[0][atom_k], -vkx);
                atomicAdd(&S.force[1][atom_k], -vky);
                atomicAdd(&S.force[2][atom_k], -vkz);
            }
            // lanes of one centre are contiguous: one wave sum per centre present in this step
            {
                const int b_first = lane_read(bsel, 0);
                const int b_last = lane_read(bsel, min(63, total - base - 1));
                for (int bb = b_first; bb <= b_last; ++bb) {
                    const bool mine = ok && (bsel == bb);
                    const float sx = group_sum_to_last_lane(mine ? cix : 0.f, 6);
                    const float sy = group_sum_to_last_lane(mine ? ciy : 0.f, 6);
                    const float sz = group_sum_to_last_lane(mine ? ciz : 0.f, 6);
                    if (lane == 63) {
                        S.force[0][c0 + bb] += sx;
                        S.force[1][c0 + bb] += sy;
                        S.force[2][c0 + bb] += sz;
                    }
                }
            }
        }
        wave_lds_fence();

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
    const unsigned blocks = (static_cast<unsigned>(n_mols) + 3u) / 4u;
    aev_bwd_small_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ);
    return hipGetLastError();
}

}  // namespace khan
