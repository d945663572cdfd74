// AEV forward for molecules of up to 64 atoms (float32): one wavefront per molecule.
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
//            four entries per trip, and stores 16 finished floats per (centre, type).
//   phase 1  the triples (centre; j<k) of the six centres are enumerated in (centre, type-pair)
//            order, each segment padded to an even length, and dealt one per lane.  A lane computes
//            what depends on the triple alone: the 8 angular factors (1+cos(theta-theta_t))^8 and the
//            4 radial factors 2^-7 f_C f_C exp(-eta (rho-Rs_s)^2).  12 floats go to LDS.
//   phase 2  lanes = (half, theta_t, Rs_s).  The halves take alternate records; a lane reads A_t and
//            G_s of its record and does one FMA into a register.  Segment boundaries are a bit mask
//            held in scalar registers; at a boundary the halves are added and 32 floats are stored
//            straight to the row in HBM.  Segments without triples are stored as zeros at the end.
// No atomics and no pre-zeroed output.  A centre with more than 32 angular neighbours (the 3.1 A
// sphere holds about 25 atoms at the densest packings tested) is redone by the general-shape
// per-centre routine.  Semantics: gpu_featurizer/kernel_cpu.cpp:406-537.
#include "aev_small_common.h"

namespace khan {

namespace {

struct __align__(16) SmallLds {
    float4 atom[64];            // x, y, z, type (sorted order)
    float4 nbr[kB][kCapA];      // unit vector (centre minus partner)/r, and r
    float nbr_fc[kB][kCapA];    // f_C(r, A_Rc)
    float2 rad[64];             // (r, f_C(r, R_Rc)); group g of a scan step owns [g*W, (g+1)*W)
    float rec[64][12];          // phase-1 records: A_0..7, G_0..3
    SegDesc seg[64];            // non-empty segments of the batch, in order
    unsigned bits[kBitWords];   // bit per triple slot: a segment starts here
    int nA[kB][4];              // angular partners per type, per centre of the batch
    int nR[4][4];               // radial partners per type, per group of the scan step
};

__global__ __launch_bounds__(64 * kWavesPerBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void aev_fwd_small_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<float> out)
{
    __shared__ SmallLds lds_all[kWavesPerBlock];
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int mol = blockIdx.x * kWavesPerBlock + wave;
    if (mol >= n_mols) return;
    const int n = uniform(MACs[mol]);
    const int off = uniform(MOs[mol]);
    if (n <= 0 || n > 64) return;                 // larger molecules belong to the general kernel
    SmallLds& S = lds_all[wave];
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
        rowbits = reinterpret_cast<unsigned long long>(out.p[type] + static_cast<size_t>(SIs[off + lane]) * kFeats);
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
    S.atom[lane] = make_float4(x, y, z, __int_as_float(type));
    auto row_of = [&](int sorted_lane) -> float* {     // sorted_lane is wave-uniform
        const unsigned lo = static_cast<unsigned>(lane_read(rp_lo, sorted_lane));
        const unsigned hi = static_cast<unsigned>(lane_read(rp_hi, sorted_lane));
        return reinterpret_cast<float*>((static_cast<unsigned long long>(hi) << 32) | lo);
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

    // segment-table lanes: lane = centre-in-batch * 10 + type-pair index (HH HC HN HO CC CN CO NN NO OO)
    const int seg_b = lane / kNumPairBlocks, seg_pt = lane - seg_b * kNumPairBlocks;
    const int seg_a = seg_pt < 4 ? 0 : seg_pt < 7 ? 1 : seg_pt < 9 ? 2 : 3;
    const int seg_bt = seg_pt < 4 ? seg_pt : seg_pt < 7 ? seg_pt - 3 : seg_pt < 9 ? seg_pt - 5 : 3;

    const float inv_rc_R = 1.0f / kR_Rc_f, inv_rc_A = 1.0f / kA_Rc_f;
    const float kRadExp = -kR_eta_f * 1.44269504088896340736f;   // exp(-eta d^2) = exp2(kRadExp d^2)
    const float kAngExp = -kA_eta_f * 1.44269504088896340736f;
    const int ang_t = L.ts >> 2, ang_s = L.ts & 3;
    wave_lds_fence();

    for (int c0 = 0; c0 < n; c0 += kB) {
        const int nb = min(kB, n - c0);
        unsigned overflow = 0;

        // ------------------------------------------------ scan steps: G centres x W partners
        for (int b0 = 0; b0 < nb; b0 += G) {
            const int b = b0 + grp;                      // centre-in-batch of this lane's group
            const int i = c0 + b;
            const bool centre_ok = b < nb;
            const float4 ai = S.atom[centre_ok ? i : 0];
            const float4 aj = S.atom[jl];
            const float dx = ai.x - aj.x, dy = ai.y - aj.y, dz = ai.z - aj.z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool valid = centre_ok && (jl < n) && (jl != i);
            const bool inR = valid && (r < kR_Rc_f);
            const bool inA = valid && (r < kA_Rc_f);
            const unsigned long long mR = wave_ballot(inR), mA = wave_ballot(inA);
            const bool fits = popc64(mA & sub_mask) <= kCapA;
            if (inR) S.rad[grp * W + popc64(mR & ltg_mask)] = make_float2(r, cutoff_poly(r * inv_rc_R));
            if (inA && fits) {
                const int pos = popc64(mA & ltg_mask);
                const float inv = __builtin_amdgcn_rcpf(r);
                S.nbr[centre_ok ? b : 0][pos] = make_float4(dx * inv, dy * inv, dz * inv, r);
                S.nbr_fc[centre_ok ? b : 0][pos] = cutoff_poly(r * inv_rc_A);
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
                if (cb < nb) S.nA[cb][cl_a] = (popc64(mA & cl_sub) <= kCapA) ? popc64(mA & cl_mask) : 0;
                S.nR[cl_g][cl_a] = cntR;
            }
            // largest radial count of each type over the groups of this step (lanes 0..15 hold them)
            int mx = cntR;
            mx = max(mx, __builtin_amdgcn_update_dpp(0, mx, 0x124, 0xf, 0xf, false));   // row_ror:4
            mx = max(mx, __builtin_amdgcn_update_dpp(0, mx, 0x128, 0xf, 0xf, false));   // row_ror:8
            const int mxR[4] = {lane_read(mx, 0), lane_read(mx, 1), lane_read(mx, 2), lane_read(mx, 3)};
            wave_lds_fence();

            // ---- radial features of the G centres of this step
            {
                const int4 cn = *reinterpret_cast<const int4*>(S.nR[rg_g]);
                const float2* list = &S.rad[rg_g * W];
                const int cb = b0 + rg_g;
                const int ci = min(c0 + cb, 63);
                const unsigned rlo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(ci << 2, rp_lo));
                const unsigned rhi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(ci << 2, rp_hi));
                float* row = reinterpret_cast<float*>((static_cast<unsigned long long>(rhi) << 32) | rlo);
                int obase = 0;
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const int cnt_a = a == 0 ? cn.x : a == 1 ? cn.y : a == 2 ? cn.z : cn.w;
                    float acc_r = 0.f;
                    for (int q0 = 0; q0 < mxR[a]; q0 += 4 * rg_ns) {
                        // four entries of this lane's slot per trip; slot s takes q = s, s+ns, s+2ns, ...
                        float2 e[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) e[u] = list[min(obase + q0 + u * rg_ns + rg_s, W - 1)];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const float dd = e[u].x - L.rrs;
                            const float v = __builtin_amdgcn_exp2f(kRadExp * dd * dd) * e[u].y;
                            acc_r += (q0 + u * rg_ns + rg_s < cnt_a) ? v : 0.f;   // stale entries: select
                        }
                    }
                    if (rg_ns >= 2) acc_r += __shfl_xor(acc_r, 16, 64);
                    if (rg_ns == 4) acc_r += __shfl_xor(acc_r, 32, 64);
                    if (rg_s == 0 && cb < nb) store_global(row + a * kNumRRs + (lane & 15), acc_r);
                    obase += cnt_a;
                }
            }
            wave_lds_fence();
        }

        // ------------------------------------------------ segment table of the batch
        int cnt = 0, packed = 0;
        unsigned seg_row_lo = 0, seg_row_hi = 0;          // where the segment's 32 floats go
        {
            // row of the segment's centre (every lane takes part in the lane exchange)
            const int cl = min(c0 + min(seg_b, kB - 1), 63);
            const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(cl << 2, rp_lo));
            const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(cl << 2, rp_hi));
            const unsigned long long rowp = ((static_cast<unsigned long long>(hi) << 32) | lo) +
                                            static_cast<unsigned long long>((kRadial + seg_pt * kAngBlock) * sizeof(float));
            seg_row_lo = static_cast<unsigned>(rowp);
            seg_row_hi = static_cast<unsigned>(rowp >> 32);
        }
        if (lane < nb * kNumPairBlocks) {
            const int4 nn = *reinterpret_cast<const int4*>(S.nA[seg_b]);
            const int na = sel4(seg_a, nn.x, nn.y, nn.z, nn.w);
            const int nbt = sel4(seg_bt, nn.x, nn.y, nn.z, nn.w);
            const int oa = sel4(seg_a, 0, nn.x, nn.x + nn.y, nn.x + nn.y + nn.z);
            const int ob = sel4(seg_bt, 0, nn.x, nn.x + nn.y, nn.x + nn.y + nn.z);
            const bool same = seg_a == seg_bt;
            cnt = same ? (na * (na - 1)) / 2 : na * nbt;
            packed = seg_b | (oa << 3) | (ob << 9) | (na << 15) | (same ? (1 << 21) : 0) | (seg_pt << 22);
        }
        const int padded = (cnt + 1) & ~1;
        const int incl = scan_add(padded);
        const int start = incl - padded;
        const int total = lane_read(incl, 63);            // triple slots in this batch (even)
        const unsigned long long nonempty = wave_ballot(cnt > 0);
        for (int w = lane; w < kBitWords; w += 64) S.bits[w] = 0u;
        wave_lds_fence();
        if (cnt > 0) {
            SegDesc d;
            d.start_cnt = start | (cnt << 12);
            d.packed = packed;
            d.row_lo = seg_row_lo;
            d.row_hi = seg_row_hi;
            S.seg[popc64(nonempty & lt_mask)] = d;
            atomicOr(&S.bits[start >> 5], 1u << (start & 31));
        }
        wave_lds_fence();

        // ------------------------------------------------ phases 1 and 2, 64 triple slots at a time
        float acc = 0.f;            // partial sums of the open segment
        unsigned cur_lo = 0, cur_hi = 0;   // where the open segment's 32 floats go (wave-uniform)
        int carry = 0;              // non-empty segments that start before this step
        // closes the open segment: the halves are added and 32 floats go straight to the row
        auto flush = [&]() {
            const float tot = half_wave_sum(acc);
            float* dst = reinterpret_cast<float*>((static_cast<unsigned long long>(cur_hi) << 32) | cur_lo);
            if (lane < 32) store_global(dst + lane, tot);
        };

        for (int base = 0; base < total; base += 64) {
            const unsigned w0 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[base >> 5])));
            const unsigned w1 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[(base >> 5) + 1])));
            const unsigned long long starts = (static_cast<unsigned long long>(w1) << 32) | w0;
            const int ord = carry + popc64(starts & (lt_mask | lane_bit)) - 1;
            carry += popc64(starts);
            const SegDesc d = S.seg[max(ord, 0)];
            const int slot = base + lane;
            const int q = slot - (d.start_cnt & 0xfff);
            const bool ok = (slot < total) && (q >= 0) && (q < (d.start_cnt >> 12));

            // decode q -> (j,k) inside the centre's type-sorted list
            int bsel = d.packed & 7;
            const int oa = (d.packed >> 3) & 63, ob = (d.packed >> 9) & 63, na = (d.packed >> 15) & 63;
            int kl, jl2;
            if ((d.packed >> 21) & 1) {                     // same type: pairs jl < kl, kl-major
                kl = static_cast<int>((1.0f + __builtin_amdgcn_sqrtf(8.0f * static_cast<float>(q) + 1.0f)) * 0.5f);
                if ((kl * (kl - 1)) / 2 > q) --kl;
                if (((kl + 1) * kl) / 2 <= q) ++kl;
                jl2 = q - (kl * (kl - 1)) / 2;
            } else {                                        // q = kl * n_a + jl
                kl = static_cast<int>((static_cast<float>(q) + 0.5f) * __builtin_amdgcn_rcpf(static_cast<float>(na)));
                jl2 = q - kl * na;
            }
            int j = oa + jl2, k = ob + kl;
            if (!ok) {
                j = 0;
                k = 0;
                bsel = 0;
            }
            const float4 vj = S.nbr[bsel][j], vk = S.nbr[bsel][k];
            const float fj = S.nbr_fc[bsel][j], fk = S.nbr_fc[bsel][k];

            float c = vj.x * vk.x + vj.y * vk.y + vj.z * vk.z;
            c = fminf(fmaxf(c, -1.0f), 1.0f);
            const float cx = vj.y * vk.z - vj.z * vk.y;
            const float cy = vj.z * vk.x - vj.x * vk.z;
            const float cz = vj.x * vk.y - vj.y * vk.x;
            const float s = __builtin_amdgcn_sqrtf(cx * cx + cy * cy + cz * cz);
            float Af[8];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                Af[t] = pow8(fmaf(s, static_cast<float>(kSinTheta[t]), fmaf(c, static_cast<float>(kCosTheta[t]), 1.0f)));
            const float rho = 0.5f * (vj.w + vk.w);
            const float P = 0.0078125f * fj * fk;
            float Gf[4];
#pragma unroll
            for (int sidx = 0; sidx < 4; ++sidx) {
                const float dd = rho - kA_Rs_f[sidx];
                // padding slots read whatever sits in the list: select, do not multiply, so that a
                // stray NaN cannot reach the sums
                Gf[sidx] = ok ? __builtin_amdgcn_exp2f(kAngExp * dd * dd) * P : 0.f;
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) Af[t] = ok ? Af[t] : 0.f;
            float4* recp = reinterpret_cast<float4*>(S.rec[lane]);
            recp[0] = make_float4(Af[0], Af[1], Af[2], Af[3]);
            recp[1] = make_float4(Af[4], Af[5], Af[6], Af[7]);
            recp[2] = make_float4(Gf[0], Gf[1], Gf[2], Gf[3]);
            wave_lds_fence();

            // phase 2: lane = (half, theta_t, Rs_s); the halves take alternate records.  Records past
            // `total` in the last step are zeros, so whole groups of eight pairs can always be run.
            const int npairs = min(64, total - base) >> 1;
            const float* pa = &S.rec[L.half][ang_t];
            const float* pg = &S.rec[L.half][8 + ang_s];
            unsigned long long mm = starts;
            if (base == 0) {            // the batch's first segment opens here; nothing to close
                cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d.row_lo), 0));
                cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d.row_hi), 0));
                mm &= ~1ull;
            }
            auto load8 = [&](int q0, float (&av)[8], float (&gv)[8]) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    av[u] = pa[(q0 + u) * 24];
                    gv[u] = pg[(q0 + u) * 24];
                }
            };
            auto run8 = [&](int q0, const float (&av)[8], const float (&gv)[8]) {
                const unsigned m16 = static_cast<unsigned>(mm) & 0xffffu;     // this group's 16 slots
                mm >>= 16;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (__builtin_expect((m16 >> (2 * u)) & 1u, 0)) {
                        // a segment starts at record pair q0+u: close the open one, open the new one
                        flush();
                        int first = 2 * (q0 + u);
                        asm volatile("" : "+s"(first));      // keeps the lane reads inside this branch
                        cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d.row_lo), first));
                        cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d.row_hi), first));
                        acc = 0.f;
                    }
                    acc = fmaf(av[u], gv[u], acc);
                }
            };
            // eight record pairs per group, the next group's LDS reads in flight while one is summed
            float a0[8], g0[8], a1[8], g1[8];
            load8(0, a0, g0);
            for (int q0 = 0; q0 < npairs; q0 += 16) {
                const bool more1 = q0 + 8 < npairs;
                if (more1) load8(q0 + 8, a1, g1);
                run8(q0, a0, g0);
                if (more1) {
                    if (q0 + 16 < npairs) load8(q0 + 16, a0, g0);
                    run8(q0 + 8, a1, g1);
                }
            }
            wave_lds_fence();
        }
        if (total > 0) flush();

        // ------------------------------------------------ segments without triples are zeros
        {
            const unsigned long long empty = ~nonempty;
            for (int b = 0; b < nb; ++b) {
                const unsigned eb = static_cast<unsigned>(empty >> (b * kNumPairBlocks)) & 0x3ffu;
                if (eb == 0u) continue;
                float* row = row_of(c0 + b) + kRadial;
#pragma unroll
                for (int pp = 0; pp < 5; ++pp) {
                    if (((eb >> (2 * pp)) & 3u) != 0u) {
                        const int pt = 2 * pp + L.half;
                        if ((eb >> pt) & 1u) store_global(row + pt * kAngBlock + L.ts, 0.f);
                    }
                }
            }
        }

        // ------------------------------------------------ centres whose list overflowed
        if (overflow) {
            __threadfence();
            for (int b = 0; b < nb; ++b) {
                if (overflow & (1u << b)) {
                    const int i_orig = lane_read(orig, c0 + b);
                    fwd_center_generic<float>(L, lane, X, Y, Z, A, off, n, i_orig,
                                              reinterpret_cast<float*>(S.rec), row_of(c0 + b));
                }
            }
            wave_lds_fence();
        }
    }
}

}  // namespace

hipError_t launch_fwd_small_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                const int32_t* SIs, Buckets<float> out, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + kWavesPerBlock - 1u) / kWavesPerBlock;
    aev_fwd_small_kernel<<<dim3(blocks), dim3(64 * kWavesPerBlock), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, out);
    return hipGetLastError();
}

}  // namespace khan
