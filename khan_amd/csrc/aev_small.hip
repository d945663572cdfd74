// AEV forward for molecules of up to 64 atoms (float32): one wavefront per molecule.
//
// Layout of the work inside a wavefront
//   * the molecule lives in registers, one atom per lane, lanes ordered by atom type (a 4-bin
//     counting sort with ballots), so every neighbour list built in lane order is type-sorted and an
//     unordered type pair (a<=b) owns a contiguous range of (j,k) pairs;
//   * centres are taken six at a time.  For each centre the 64 lanes test all partners at once; the
//     partners inside the radial cutoff go to a (r, f_C) list and the 64 lanes, as (type, shell)
//     slots, walk their own type's part of that list: the radial 64 floats of the row are produced
//     in registers and stored with one coalesced 256-byte store.  Partners inside the angular cutoff
//     go to a per-centre list of unit vectors in LDS;
//   * phase 1: the triples (centre; j<k) of the six centres are enumerated in (centre, type-pair)
//     order, padded to even counts, and dealt one per lane.  A lane computes everything that depends
//     on the triple alone -- the 8 angular factors (1+cos(theta-theta_t))^8 and the 4 radial factors
//     2^-7 f_C f_C exp(-eta (rho-Rs_s)^2) -- 12 floats, written to LDS;
//   * phase 2: lanes become (half, theta_t, Rs_s) slots.  The two halves take alternate records; a
//     lane reads A_t and G_s of its record and does one FMA into a register accumulator.  When the
//     (centre, type-pair) segment changes, the halves are added and the 32 values are stored straight
//     to the row in HBM; empty segments are stored as zeros.  No atomics, no output pre-zeroing.
//
// A centre with more than 32 angular neighbours (not reachable with physical geometries: the angular
// cutoff sphere of 3.1 A holds about 25 atoms at the densest packing seen) is redone by the
// general-shape per-centre routine.  Semantics: gpu_featurizer/kernel_cpu.cpp:406-537.
#include "aev_generic_center.h"

namespace khan {

namespace {

constexpr int kB = 6;                          // centres per batch
constexpr int kCapA = 32;                      // angular neighbours kept per centre
constexpr int kSegLanes = kB * kNumPairBlocks; // 60 (centre, type-pair) segments per batch

struct __align__(16) SegDesc {
    int start;       // first triple slot of the segment inside the batch (even)
    int cnt;         // triples in the segment (the slot range is padded to an even length)
    int packed;      // centre-in-batch | list offset of type a | offset of type b | n_a | a==b
    float rcp_na;    // 1 / n_a
};

struct __align__(16) SmallLds {
    float4 nbr[kB][kCapA];      // unit vector centre->partner (centre minus partner) and distance
    float nbr_fc[kB][kCapA];    // f_C(r, A_Rc)
    float2 rad[64];             // (r, f_C(r, R_Rc)) of the current centre's radial partners
    float rec[64][12];          // phase-1 records: A_0..7, G_0..3
    SegDesc seg[64];
    int marker[64];
    int nA[kB][4];              // angular partners per type, per centre
};

__device__ __forceinline__ float lane_read(float v, int src_lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}
__device__ __forceinline__ int lane_read(int v, int src_lane) { return __builtin_amdgcn_readlane(v, src_lane); }

__device__ __forceinline__ float lane_push(int dest_lane, float v)   // value lands in lane dest_lane
{
    return __int_as_float(__builtin_amdgcn_ds_permute(dest_lane << 2, __float_as_int(v)));
}
__device__ __forceinline__ int lane_push(int dest_lane, int v) { return __builtin_amdgcn_ds_permute(dest_lane << 2, v); }

__device__ __forceinline__ int scan_add(int v, int lane)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(v, d, 64);
        if (lane >= d) v += y;
    }
    return v;
}
__device__ __forceinline__ int scan_max(int v, int lane)
{
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int y = __shfl_up(v, d, 64);
        if (lane >= d) v = max(v, y);
    }
    return v;
}

__device__ __forceinline__ float pow8(float b)
{
    const float b2 = b * b, b4 = b2 * b2;
    return b4 * b4;
}

__device__ __forceinline__ int sel4(int a, int v0, int v1, int v2, int v3)
{
    return a == 0 ? v0 : a == 1 ? v1 : a == 2 ? v2 : v3;
}

__global__ __launch_bounds__(256) void aev_fwd_small_kernel(
    const float* __restrict__ X, const float* __restrict__ Y, const float* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<float> out)
{
    __shared__ SmallLds lds_all[4];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mol = blockIdx.x * 4 + wave;
    if (mol >= n_mols) return;
    const int n = __builtin_amdgcn_readfirstlane(MACs[mol]);
    const int off = __builtin_amdgcn_readfirstlane(MOs[mol]);
    if (n <= 0 || n > 64) return;                 // larger molecules belong to the general kernel
    SmallLds& S = lds_all[wave];
    const LaneConsts<float> L = lane_consts<float>(lane);
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

    // ---- one atom per lane, then lanes reordered by type
    const bool have = lane < n;
    float x = 0.f, y = 0.f, z = 0.f;
    int type = 0, orig = lane;
    float* rowp = nullptr;
    if (have) {
        x = X[off + lane];
        y = Y[off + lane];
        z = Z[off + lane];
        type = fold_type(A[off + lane]);
        rowp = out.p[type] + static_cast<size_t>(SIs[off + lane]) * kFeats;
    }
    unsigned long long tmask[4];
    int tcount[4], tbase[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        tmask[a] = wave_ballot(have && type == a);
        tcount[a] = __popcll(tmask[a]);
    }
    tbase[0] = 0;
    tbase[1] = tcount[0];
    tbase[2] = tbase[1] + tcount[1];
    tbase[3] = tbase[2] + tcount[2];
    int dest = lane;    // lanes without an atom keep their place, so the map is a permutation
    if (have) {
        const unsigned long long mine = type == 0 ? tmask[0] : type == 1 ? tmask[1] : type == 2 ? tmask[2] : tmask[3];
        dest = sel4(type, tbase[0], tbase[1], tbase[2], tbase[3]) + __popcll(mine & lt_mask);
    }
    x = lane_push(dest, x);
    y = lane_push(dest, y);
    z = lane_push(dest, z);
    type = lane_push(dest, type);
    orig = lane_push(dest, orig);
    {
        const unsigned long long rp = reinterpret_cast<unsigned long long>(rowp);
        const int lo = lane_push(dest, static_cast<int>(rp & 0xffffffffull));
        const int hi = lane_push(dest, static_cast<int>(rp >> 32));
        rowp = reinterpret_cast<float*>((static_cast<unsigned long long>(static_cast<unsigned>(hi)) << 32) |
                                        static_cast<unsigned>(lo));
    }
    const int rp_lo = static_cast<int>(reinterpret_cast<unsigned long long>(rowp) & 0xffffffffull);
    const int rp_hi = static_cast<int>(reinterpret_cast<unsigned long long>(rowp) >> 32);
    // masks of the sorted lanes that hold each type
    unsigned long long smask[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
        smask[a] = (tcount[a] == 0) ? 0ull : ((tcount[a] >= 64 ? ~0ull : ((1ull << tcount[a]) - 1ull)) << tbase[a]);

    auto row_of = [&](int sorted_lane) -> float* {
        const unsigned lo = static_cast<unsigned>(lane_read(rp_lo, sorted_lane));
        const unsigned hi = static_cast<unsigned>(lane_read(rp_hi, sorted_lane));
        return reinterpret_cast<float*>((static_cast<unsigned long long>(hi) << 32) | lo);
    };

    // per-lane constants of the segment table: lane = centre-in-batch * 10 + type-pair index
    const int seg_b = lane / kNumPairBlocks, seg_pt = lane - seg_b * kNumPairBlocks;
    // type pair (a <= b) of pair index pt:  HH HC HN HO CC CN CO NN NO OO
    const int seg_a = seg_pt < 4 ? 0 : seg_pt < 7 ? 1 : seg_pt < 9 ? 2 : 3;
    const int seg_bt = seg_pt < 4 ? seg_pt : seg_pt < 7 ? seg_pt - 3 : seg_pt < 9 ? seg_pt - 5 : 3;

    const float inv_rc_R = 1.0f / kR_Rc_f, inv_rc_A = 1.0f / kA_Rc_f;
    const float kRadExp = -kR_eta_f * 1.44269504088896340736f;   // exp(-eta d^2) = exp2(kRadExp d^2)
    const float kAngExp = -kA_eta_f * 1.44269504088896340736f;
    const int ang_t = L.ts >> 2, ang_s = L.ts & 3;

    for (int c0 = 0; c0 < n; c0 += kB) {
        const int nb = min(kB, n - c0);
        unsigned overflow = 0;

        // ------------------------------------------------ scan + radial part, centre by centre
        for (int b = 0; b < nb; ++b) {
            const int i = c0 + b;
            const float dx = lane_read(x, i) - x, dy = lane_read(y, i) - y, dz = lane_read(z, i) - z;
            const float r = sqrtf(dx * dx + dy * dy + dz * dz);
            const bool valid = have && (lane != i);
            const bool inR = valid && (r < kR_Rc_f);
            const bool inA = valid && (r < kA_Rc_f);
            const unsigned long long mR = wave_ballot(inR), mA = wave_ballot(inA);
            if (inR) S.rad[__popcll(mR & lt_mask)] = make_float2(r, 0.5f * cospif(r * inv_rc_R) + 0.5f);
            const int cntA = __popcll(mA);
            const bool fits = cntA <= kCapA;
            if (!fits) overflow |= 1u << b;
            if (inA && fits) {
                const int pos = __popcll(mA & lt_mask);
                const float inv = __builtin_amdgcn_rcpf(r);
                S.nbr[b][pos] = make_float4(dx * inv, dy * inv, dz * inv, r);
                S.nbr_fc[b][pos] = 0.5f * cospif(r * inv_rc_A) + 0.5f;
            }
            {
                const int a0 = __popcll(mA & smask[0]), a1 = __popcll(mA & smask[1]),
                          a2 = __popcll(mA & smask[2]), a3 = __popcll(mA & smask[3]);
                if (lane < 4) S.nA[b][lane] = fits ? sel4(lane, a0, a1, a2, a3) : 0;
            }
            const int r0 = __popcll(mR & smask[0]), r1 = __popcll(mR & smask[1]),
                      r2 = __popcll(mR & smask[2]), r3 = __popcll(mR & smask[3]);
            wave_lds_fence();
            {
                // lane = (partner type, shell): walk this type's part of the radial list
                const int my_n = sel4(L.rtype, r0, r1, r2, r3);
                const int my_o = sel4(L.rtype, 0, r0, r0 + r1, r0 + r1 + r2);
                const int max_n = max(max(r0, r1), max(r2, r3));
                float acc_rad = 0.f;
                for (int q = 0; q < max_n; ++q) {
                    if (q < my_n) {
                        const float2 e = S.rad[my_o + q];
                        const float d = e.x - L.rrs;
                        acc_rad += __builtin_amdgcn_exp2f(kRadExp * d * d) * e.y;
                    }
                }
                row_of(i)[lane] = acc_rad;
            }
            wave_lds_fence();
        }

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
            packed = seg_b | (oa << 3) | (ob << 9) | (na << 15) | (same ? (1 << 21) : 0);
            rcp_na = na > 0 ? 1.0f / static_cast<float>(na) : 0.f;
        }
        const int padded = (cnt + 1) & ~1;
        const int incl = scan_add(padded, lane);
        const int start = incl - padded;
        const int total = lane_read(incl, 63);            // triple slots in this batch (even)
        {
            SegDesc d;
            d.start = start;
            d.cnt = cnt;
            d.packed = packed;
            d.rcp_na = rcp_na;
            S.seg[lane] = d;
        }
        wave_lds_fence();

        // ------------------------------------------------ phases 1 and 2, 64 triple slots at a time
        int cur = -1;          // segment whose sum is in `acc` (-1: none yet in this batch)
        float acc = 0.f;
        auto store_segment = [&](int sgi, float v) {
            const int bb = sgi / kNumPairBlocks, pt = sgi - bb * kNumPairBlocks;
            float* row = row_of(c0 + bb);
            if (lane < 32) row[kRadial + pt * kAngBlock + lane] = v;
        };
        auto flush_until = [&](int next) {      // close `cur`, zero-fill the empty segments up to `next`
            if (cur >= 0) store_segment(cur, acc + __shfl_xor(acc, 32, 64));
            for (int s2 = cur + 1; s2 < next; ++s2) store_segment(s2, 0.f);
        };

        for (int base = 0; base < total; base += 64) {
            // which segment does each of the 64 slots belong to: segment starts are marked, then
            // carried forward with a max-scan (segment ids grow with the slot index)
            S.marker[lane] = 0;
            wave_lds_fence();
            if (cnt > 0) {
                const int rel = start - base;
                if (rel >= 0 && rel < 64) S.marker[rel] = lane + 1;
                else if (rel < 0 && start + padded > base) S.marker[0] = lane + 1;
            }
            wave_lds_fence();
            const int seg_of_lane = max(scan_max(S.marker[lane], lane) - 1, 0);
            const SegDesc d = S.seg[seg_of_lane];
            const int slot = base + lane;
            const int q = slot - d.start;
            const bool ok = (slot < total) && (q >= 0) && (q < d.cnt);

            // decode q -> (j,k) inside the centre's type-sorted list
            int bsel = d.packed & 7;
            const int oa = (d.packed >> 3) & 63, ob = (d.packed >> 9) & 63, na = (d.packed >> 15) & 63;
            int kl, jl;
            if ((d.packed >> 21) & 1) {                     // same type: pairs jl < kl, kl-major
                kl = static_cast<int>((1.0f + __builtin_amdgcn_sqrtf(8.0f * static_cast<float>(q) + 1.0f)) * 0.5f);
                if ((kl * (kl - 1)) / 2 > q) --kl;
                if (((kl + 1) * kl) / 2 <= q) ++kl;
                jl = q - (kl * (kl - 1)) / 2;
            } else {                                        // q = kl * n_a + jl
                kl = static_cast<int>((static_cast<float>(q) + 0.5f) * d.rcp_na);
                jl = q - kl * na;
            }
            int j = oa + jl, k = ob + kl;
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

            // phase 2: lane = (half, theta_t, Rs_s); the halves take alternate records
            const int npairs = min(64, total - base) >> 1;
            const float* pa = &S.rec[L.half][ang_t];
            const float* pg = &S.rec[L.half][8 + ang_s];
            for (int qq = 0; qq < npairs; ++qq) {
                const int sg = lane_read(seg_of_lane, 2 * qq);
                if (sg != cur) {
                    flush_until(sg);
                    cur = sg;
                    acc = 0.f;
                }
                acc = fmaf(pa[qq * 24], pg[qq * 24], acc);
            }
            wave_lds_fence();
        }
        flush_until(nb * kNumPairBlocks);

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
        }
    }
}

}  // namespace

hipError_t launch_fwd_small_f32(const float* X, const float* Y, const float* Z, const int32_t* A,
                                const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                                const int32_t* SIs, Buckets<float> out, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const unsigned blocks = (static_cast<unsigned>(n_mols) + 3u) / 4u;
    aev_fwd_small_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, out);
    return hipGetLastError();
}

}  // namespace khan
