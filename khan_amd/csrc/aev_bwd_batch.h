// Pieces of the one-wavefront AEV backward pass shared by the small-molecule kernel (one wavefront per
// molecule) and the medium-molecule kernel (four wavefronts per molecule): the pooled neighbour lists of a
// batch of centres, the radial pull of one (centre, partner) pair, and the round-robin angular walk.
#pragma once
#include "aev_small_common.h"

namespace khan {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f* global_v4f_ptr;

constexpr int kBlockStride = 36;   // floats between staged 32-float blocks: rotates the LDS banks

// per-wavefront LDS of a batch: the centres' angular partner lists laid end to end (at most 64 entries)
// and their rows' angular upstream values
struct __align__(16) BwdPool {
    float4 nbr[64];                               // unit vector (centre minus partner)/r, and r
    float4 facc[64];                              // force on each list entry from its centre's row
    float2 nbr_fc[64];                            // f_C(r, A_Rc) and its derivative in r
    float gst[kB * kNumPairBlocks * kBlockStride];   // staged upstream blocks [centre][type pair][32]
    unsigned char nbr_idx[64];                    // sorted position of the partner
};

__device__ __forceinline__ int sel6(int b, int v0, int v1, int v2, int v3, int v4, int v5)
{
    return b == 0 ? v0 : b == 1 ? v1 : b == 2 ? v2 : b == 3 ? v3 : b == 4 ? v4 : v5;
}

// Radial part of one (centre, partner) pair: sum over the 16 shells of g e (f_C' - 2 eta d f_C), divided
// by r.  The result times (x_i - x_j) is the pair's pull on the centre (and minus that on the partner).
// `grow` is the centre's upstream row, `tj` the partner's type, `inv` = 1/r.
__device__ __forceinline__ float bwd_radial_pair(const float* grow, int tj, float r, float inv)
{
    const float inv_rc_R = 1.0f / kR_Rc_f;
    const float kRadExp = -kR_eta_f * 1.44269504088896340736f;
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
    return Gsum * inv;           // dE/dr / r
}

// Writes the angular part (80 x 16 bytes) of up to kB upstream rows, fetched as chunk `lane` (st0) and
// chunk 64 + lane (st1, lanes 0..15) of each row, into the pool: chunk c of a row = block c/8, part c%8.
__device__ __forceinline__ void bwd_stage_blocks(BwdPool& P, int lane, int nb, const v4f (&st0)[kB], const v4f (&st1)[kB])
{
#pragma unroll
    for (int b = 0; b < kB; ++b) {
        if (b < nb) {
            float* blk = &P.gst[b * kNumPairBlocks * kBlockStride];
            *reinterpret_cast<v4f*>(blk + (lane >> 3) * kBlockStride + (lane & 7) * 4) = st0[b];
            if (lane < 16) *reinterpret_cast<v4f*>(blk + (8 + (lane >> 3)) * kBlockStride + (lane & 7) * 4) = st1[b];
        }
    }
}

// Angular walk of a batch.  Lane = list entry `lane` of the pool, belonging to centre `bs` of the batch
// whose list starts at slot `pb` and has `m` entries (`live` = the lane has an entry).  In round d the
// entry pairs with entry (e + d) mod m of the same centre; after m/2 rounds every unordered pair has
// been visited once.  The force on the partner k goes to P.facc[k] by plain read-add-write (the k of a
// centre are distinct within a round); the force on the lane's own entry is kept in registers.
// Returns the lane's total: P.facc[lane] + own (zero for lanes without an entry).
// `type_of(sorted position)` gives an atom's type.
template <typename TypeOf>
__device__ __forceinline__ float4 bwd_angular_rounds(BwdPool& pool, int lane, bool live, int bs, int pb, int m,
                                                     TypeOf type_of)
{
    const float kAngExp = -kA_eta_f * 1.44269504088896340736f;
    const int e = live ? lane - pb : 0;
    // rounds: d = 1 .. (m-1)/2 for every lane; when m is even one more round for the lower half
    const int full = (m - 1) >> 1;
    const int rounds = live ? full + ((((m & 1) == 0) && (e < (m >> 1))) ? 1 : 0) : 0;
    const int max_rounds = wave_max(rounds);
    const int self = live ? lane : 0;
    const float4 vj = pool.nbr[self];
    const float2 fj = pool.nbr_fc[self];
    const int tj = type_of(pool.nbr_idx[self]);
    const float inv_rj = __builtin_amdgcn_rcpf(vj.w);
    const float* gbase = &pool.gst[bs * kNumPairBlocks * kBlockStride];
    float ajx = 0.f, ajy = 0.f, ajz = 0.f;           // force on j, kept in registers

    for (int d = 1; d <= max_rounds; ++d) {
        const bool act = d <= rounds;
        int k = e + d;
        k -= (k >= m) ? m : 0;
        const int ks = act ? pb + k : 0;
        const float4 vk = pool.nbr[ks];
        const float2 fk = pool.nbr_fc[ks];
        const int tk = type_of(pool.nbr_idx[ks]);
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
            float4 fk_acc = pool.facc[ks];
            fk_acc.x = fmaf(-Fk, vk.x, fmaf(-ik, fmaf(-c, vk.x, vj.x), fk_acc.x));
            fk_acc.y = fmaf(-Fk, vk.y, fmaf(-ik, fmaf(-c, vk.y, vj.y), fk_acc.y));
            fk_acc.z = fmaf(-Fk, vk.z, fmaf(-ik, fmaf(-c, vk.z, vj.z), fk_acc.z));
            pool.facc[ks] = fk_acc;
        }
        wave_lds_fence();
    }

    float4 f = pool.facc[self];
    f.x = live ? f.x + ajx : 0.f;
    f.y = live ? f.y + ajy : 0.f;
    f.z = live ? f.z + ajz : 0.f;
    return f;
}

}  // namespace khan
