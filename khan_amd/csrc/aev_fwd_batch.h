// Angular part of the one-wavefront AEV forward pass for a batch of up to six centres whose
// type-sorted neighbour lists are in LDS: shared by the small-molecule kernel (one wavefront per
// molecule) and the medium-molecule kernel (four wavefronts per molecule).
#pragma once
#include "aev_small_common.h"

namespace khan {

// LDS working set of one wavefront
// what the Jacobian-vector variant keeps on top of the forward working set
template <typename T, bool kJvp, int kNB, int kRadN, int kCap> struct FwdJvpLds {};
template <typename T, int kNB, int kRadN, int kCap> struct __align__(16) FwdJvpLds<T, true, kNB, kRadN, kCap> {
    typename Fast<T>::vec4 nbr_p[kNB][kCap];       // (v_centre - v_partner)/r, and its component along the unit vector: dr / r
    T nbr_dfc[kNB][kCap];                          // f_C'(r) dr, dr = change of the distance along the vectors (= nbr_p.w r)
    typename Fast<T>::vec2 rad_ab[kRadN];         // radial entries: f_C' dr, and -2 eta f_C dr
    T rec2[64][12];                               // phase-1 records: dA_0..7, H_0..3
};

// LDS working set of one wavefront, for batches of kNB centres with at most kCap angular partners each
template <typename T, bool kJvp = false, int kNB = kFB, int kRadN = 64, int kCap = kCapA>
struct __align__(16) FwdWaveLds {
    static constexpr int kCentres = kNB;
    static constexpr int kCapacity = kCap;
    static constexpr int kSegments = kNB * kNumPairBlocks;      // a segment per (centre, type pair) at most
    typename Fast<T>::vec4 nbr[kNB][kCap];     // unit vector (centre minus partner)/r, and r
    T nbr_fc[kNB][kCap];                       // f_C(r, A_Rc)
    typename Fast<T>::vec2 rad[kRadN];        // (r, f_C(r, R_Rc)) of the radial partners of a scan step's centres
    T rec[64][12];                            // phase-1 records: A_0..7, G_0..3
    SegDesc seg[kSegments];                   // non-empty segments of the batch, in order
    unsigned long long segrow[kSegments];     // where each of them puts its 32 output values (then: the empty blocks' addresses)
    unsigned bits[bit_words(kNB)];            // bit per triple slot: a segment starts here
    int nA[kNB][4];                            // angular partners per type, per centre of the batch
    FwdJvpLds<T, kJvp, kNB, kRadN, kCap> jvp;
};

// Padding slots of phase 1 read entry 0 of centre 0's list whatever it holds; their products are cancelled by a
// zero radial factor, which needs every other factor finite.  Entry 0 is either a partner written by a scan or
// what this writes once per wavefront before the first batch.
template <typename T, bool kJvp, int kNB, int kRadN, int kCap>
__device__ __forceinline__ void fwd_lds_init(FwdWaveLds<T, kJvp, kNB, kRadN, kCap>& S, int lane)
{
    if (lane == 0) {
        S.nbr[0][0] = Fast<T>::make4(T(0), T(0), T(0), T(0));
        S.nbr_fc[0][0] = T(0);
        if constexpr (kJvp) {
            S.jvp.nbr_p[0][0] = Fast<T>::make4(T(0), T(0), T(0), T(0));
            S.jvp.nbr_dfc[0][0] = T(0);
        }
    }
}

// Segment table, phases 1 and 2 and the zero fill of empty blocks for centres 0..nb-1 of a batch (nb <= kNB <= 6).
// `row_of_centre(b)` returns the address of centre b's 384-float output row; it is called by all
// lanes together, with a per-lane b.
// With kJvp the same sums are formed for the derivative of every term along the atoms' incoming vectors:
// d(A_t G_s P) = dA_t (G_s P) + A_t (dG_s P + G_s dP), two products per record instead of one.
//
// kMatrixPhase2 (float, forward only) sums the records on the matrix cores instead of the vector ALU: the sum over a
// segment's records of A_t G_s is the product of an 8 x K by a K x 4 matrix, and v_mfma_f32_16x16x4_f32 takes four
// records (K = 4) per instruction, using an 8 x 4 corner of its 16 x 16 result.  The variant exists to be measured
// against the vector form; the launcher selects it on request only.
template <bool kMatrixPhase2, typename T, bool kJvp, int kNB, int kRadN, int kCap, typename RowOfCentre>
__device__ __forceinline__ void fwd_angular_batch(FwdWaveLds<T, kJvp, kNB, kRadN, kCap>& S, const LaneConsts<T>& L, int lane, int nb,
                                                  RowOfCentre row_of_centre)
{
    static_assert(kNB * kNumPairBlocks <= 64, "one segment-table lane per (centre, type pair)");
    static_assert(!kMatrixPhase2 || (sizeof(T) == 4 && !kJvp), "the matrix-core phase 2 is float, forward only");
    typedef typename Fast<T>::vec4 vec4;
    typedef typename Fast<T>::vec2 vec2;
    const unsigned long long lane_bit = 1ull << lane;
    const unsigned long long lt_mask = lane_bit - 1ull;
    // segment-table lanes: lane = centre-in-batch * 10 + type-pair index (HH HC HN HO CC CN CO NN NO OO)
    const int seg_b = lane / kNumPairBlocks, seg_pt = lane - seg_b * kNumPairBlocks;
    const int seg_a = seg_pt < 4 ? 0 : seg_pt < 7 ? 1 : seg_pt < 9 ? 2 : 3;
    const int seg_bt = seg_pt < 4 ? seg_pt : seg_pt < 7 ? seg_pt - 3 : seg_pt < 9 ? seg_pt - 5 : 3;
    const int ang_t = L.ts >> 2, ang_s = L.ts & 3;

    // ------------------------------------------------ segment table of the batch
    int cnt = 0;
    SegDesc mine = {0u, 0u, 0u, 0u};
    unsigned seg_row_lo = 0, seg_row_hi = 0;          // where the segment's 32 floats go
    {
        // row of the segment's centre (every lane takes part: the lookup may be a lane exchange)
        const unsigned long long rowp = row_of_centre(min(seg_b, kNB - 1)) +
                                        static_cast<unsigned long long>((kRadial + seg_pt * kAngBlock) * sizeof(T));
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
        cnt = same ? (__mul24(na, na - 1) >> 1) : __mul24(na, nbt);
        mine.aj = static_cast<unsigned>((seg_b * kCap + oa) * static_cast<int>(sizeof(vec4)));
        mine.ak = static_cast<unsigned>((seg_b * kCap + ob) * static_cast<int>(sizeof(vec4)));
        // floor(2^15 / n_a) + 1 (the reciprocal is within an ulp, and 2^15 / n_a is never that close below an integer)
        const unsigned magic = static_cast<unsigned>(32768.0f * __builtin_amdgcn_rcpf(static_cast<float>(max(na, 1)))) + 1u;
        mine.div = magic | (static_cast<unsigned>(na) << 16) | (same ? (1u << 24) : 0u);
    }
    const int padded = (cnt + 1) & ~1;
    const int incl = scan_add(padded);
    const int start = incl - padded;
    const int total = kSkipAngular ? 0 : lane_read(incl, 63);            // triple slots in this batch (even)
    const unsigned long long nonempty = wave_ballot(cnt > 0);
    // (lanes past the last word write the last word again: no loop, no branch)
#pragma unroll
    for (int w0 = 0; w0 < bit_words(kNB); w0 += 64) S.bits[min(w0 + lane, bit_words(kNB) - 1)] = 0u;
    wave_lds_fence();
    if (cnt > 0) {
        mine.start_cnt = static_cast<unsigned>(start) | (static_cast<unsigned>(cnt) << 16);
        const int at = popc64(nonempty & lt_mask);
        S.seg[at] = mine;
        S.segrow[at] = (static_cast<unsigned long long>(seg_row_hi) << 32) | seg_row_lo;
        atomicOr(&S.bits[start >> 5], 1u << (start & 31));
    }
    wave_lds_fence();

    // ------------------------------------------------ phases 1 and 2, 64 triple slots at a time
    T acc = T(0);               // partial sums of the open segment
    unsigned cur_lo = 0, cur_hi = 0;   // where the open segment's 32 floats go (wave-uniform)
    int carry = 0;              // non-empty segments that start before this step
    // closes the open segment: the halves are added and 32 floats go straight to the row
    auto flush = [&]() {
        const T tot = half_wave_sum(acc);
        T* dst = reinterpret_cast<T*>((static_cast<unsigned long long>(cur_hi) << 32) | cur_lo);
        if (lane < 32) store_global(dst + lane, tot);
    };
    // matrix-core form: result element (theta_t, Rs_s) of the open segment is register t % 4 of lane 16 (t / 4) + s
    typedef float mfma_acc __attribute__((ext_vector_type(4)));
    mfma_acc macc = {0.f, 0.f, 0.f, 0.f};
    auto flush_matrix = [&]() {
        T* dst = reinterpret_cast<T*>((static_cast<unsigned long long>(cur_hi) << 32) | cur_lo);
        if (lane < 32 && (lane & 15) < 4) {
            T* p = dst + (lane >> 4) * 16 + (lane & 15);
#pragma unroll
            for (int v = 0; v < 4; ++v) store_global(p + 4 * v, static_cast<T>(macc[v]));
        }
    };

    for (int base = 0; base < total; base += 64) {
        const unsigned w0 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[base >> 5])));
        const unsigned w1 = static_cast<unsigned>(uniform(static_cast<int>(S.bits[(base >> 5) + 1])));
        const unsigned long long starts = (static_cast<unsigned long long>(w1) << 32) | w0;
        const int ord = carry + popc64(starts & (lt_mask | lane_bit)) - 1;
        carry += popc64(starts);
        const int seg_at = max(ord, 0);
        const SegDesc d = S.seg[seg_at];
        const unsigned long long d_row = S.segrow[seg_at];
        const unsigned d_row_lo = static_cast<unsigned>(d_row), d_row_hi = static_cast<unsigned>(d_row >> 32);
        const int slot = base + lane;
        const unsigned q = static_cast<unsigned>(slot) - (d.start_cnt & 0xffffu);     // "negative" = huge
        const bool ok = (slot < total) && (q < (d.start_cnt >> 16));

        // decode q -> (j,k) inside the centre's type-sorted list
        // Different types: q = kl * n_a + jl.  Same type (pairs jl < kl): the rows kl = r + 1 and kl = n_a - r - 1 of the
        // triangle are laid end to end in one row of length n_a, so the same division serves both numberings:
        // with (r, col) = divmod(q, n_a), col <= r is the pair (col, r + 1) and col > r the pair (col - r - 1, n_a - r - 1).
        const unsigned na = (d.div >> 16) & 0xffu, tri = d.div >> 24;
        const unsigned kr = __umul24(q, d.div & 0xffffu) >> 15;
        const unsigned jr = q - __umul24(kr, na);
        const unsigned k1 = kr + tri;
        const bool fold = tri && (jr >= k1);
        const unsigned kl = fold ? na - k1 : k1;
        const unsigned jl2 = fold ? jr - k1 : jr;
        // byte offsets of the two list entries (padding slots take entry 0 of the first list)
        constexpr unsigned kEntry = sizeof(vec4), kPerT = sizeof(vec4) / sizeof(T);
        const unsigned bj = ok ? d.aj + jl2 * kEntry : 0u;
        const unsigned bk = ok ? d.ak + kl * kEntry : 0u;
        const char* const nbr_bytes = reinterpret_cast<const char*>(&S.nbr[0][0]);
        const char* const fc_bytes = reinterpret_cast<const char*>(&S.nbr_fc[0][0]);
        const vec4 vj = *reinterpret_cast<const vec4*>(nbr_bytes + bj), vk = *reinterpret_cast<const vec4*>(nbr_bytes + bk);
        const T fj = *reinterpret_cast<const T*>(fc_bytes + bj / kPerT), fk = *reinterpret_cast<const T*>(fc_bytes + bk / kPerT);

        T c = vj.x * vk.x + vj.y * vk.y + vj.z * vk.z;
        c = fmin(fmax(c, T(-1)), T(1));
        const T cx = vj.y * vk.z - vj.z * vk.y;
        const T cy = vj.z * vk.x - vj.x * vk.z;
        const T cz = vj.x * vk.y - vj.y * vk.x;
        // clamped to [0, 1] like c: a coincident partner (unit vector 0/0) then gives c = -1, s = 0, the angle pi
        // that the reference arrives at through fmax/fmin/acos (kernel_cpu.cpp:514-517)
        const T s = Fast<T>::sqrt_(fmin(fmax(cx * cx + cy * cy + cz * cz, T(0)), T(1)));
        T Af[8], dAf[8];
        T dc = T(0), cot = T(0);
        T drj = T(0), drk = T(0);          // change of the two distances along the vectors
        if constexpr (kJvp) {
            // d cos = u_k.p_j + u_j.p_k - c (alpha_j + alpha_k), p = (v_i - v_partner)/r, alpha = u.p
            const char* const p_bytes = reinterpret_cast<const char*>(&S.jvp.nbr_p[0][0]);
            const vec4 pj = *reinterpret_cast<const vec4*>(p_bytes + bj), pk = *reinterpret_cast<const vec4*>(p_bytes + bk);
            dc = (vk.x * pj.x + vk.y * pj.y + vk.z * pj.z) + (vj.x * pk.x + vj.y * pk.y + vj.z * pk.z) - c * (pj.w + pk.w);
            drj = pj.w * vj.w;
            drk = pk.w * vk.w;
            cot = c * s * Fast<T>::rcp(s * s + Real<T>::kCotEps);     // c/s, zero on the line (cusp of the angle)
        }
        T bases[8];
        theta_bases<T>(c, s, bases);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const T ct = static_cast<T>(kCosTheta[t]), st = static_cast<T>(kSinTheta[t]);
            const T base = bases[t];
            if constexpr (kJvp) {
                const T b2 = base * base, b4 = b2 * b2;
                const T Am1 = b4 * b2 * base;
                Af[t] = Am1 * base;
                dAf[t] = T(8) * Am1 * fma(-cot, st, ct) * dc;
            } else {
                Af[t] = pow8(base);
                dAf[t] = T(0);
            }
        }
        const T rho = T(0.5) * (vj.w + vk.w);
        // padding slots read entry 0 of centre 0's list (finite, see fwd_lds_init): a zero radial factor,
        // selected and not multiplied in, cancels their records in phase 2
        const T P = ok ? T(0.0078125) * fj * fk : T(0);
        T Gf[4], Hf[4];
        T dP = T(0), drho = T(0);
        if constexpr (kJvp) {
            const char* const d_bytes = reinterpret_cast<const char*>(&S.jvp.nbr_dfc[0][0]);
            const T dj = *reinterpret_cast<const T*>(d_bytes + bj / kPerT), dk = *reinterpret_cast<const T*>(d_bytes + bk / kPerT);
            dP = ok ? T(0.0078125) * (dj * fk + fj * dk) : T(0);
            drho = T(0.5) * (drj + drk);
        }
#pragma unroll
        for (int sidx = 0; sidx < 4; ++sidx) {
            const T dd = rho - static_cast<T>(kA_Rs_f[sidx]);
            const T g = Fast<T>::gauss(static_cast<T>(kA_eta_f), dd);
            Gf[sidx] = g * P;
            if constexpr (kJvp) Hf[sidx] = g * fma(T(-2) * static_cast<T>(kA_eta_f) * dd * drho, P, dP);
            else Hf[sidx] = T(0);
        }
        vec4* recp = reinterpret_cast<vec4*>(S.rec[lane]);
        recp[0] = Fast<T>::make4(Af[0], Af[1], Af[2], Af[3]);
        recp[1] = Fast<T>::make4(Af[4], Af[5], Af[6], Af[7]);
        recp[2] = Fast<T>::make4(Gf[0], Gf[1], Gf[2], Gf[3]);
        if constexpr (kJvp) {
            vec4* rec2p = reinterpret_cast<vec4*>(S.jvp.rec2[lane]);
            rec2p[0] = Fast<T>::make4(dAf[0], dAf[1], dAf[2], dAf[3]);
            rec2p[1] = Fast<T>::make4(dAf[4], dAf[5], dAf[6], dAf[7]);
            rec2p[2] = Fast<T>::make4(Hf[0], Hf[1], Hf[2], Hf[3]);
        }
        wave_lds_fence();

        if constexpr (kMatrixPhase2) {
            // phase 2 on the matrix cores, four records per instruction.  Operand A (16 x 4): lane 16 k + i supplies
            // row i of record k, operand B (4 x 16): lane 16 k + j column j of record k.  Rows 0-7 are A_0..7 and
            // columns 0-3 are G_0..3; the other rows and columns take whatever follows in the record buffer, which
            // only reaches result elements outside the 8 x 4 corner.  Segments start at even records: a start in
            // the middle of a group splits it into two instructions, each with the other half's rows zeroed.
            const int nrec = min(64, total - base);
            const int ngroups = (nrec + 3) >> 2;           // records past `total` are zeros
            const float* pm = &S.rec[0][0] + (lane >> 4) * 12 + (lane & 15);
            unsigned long long mm = starts;
            if (base == 0) {
                cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d_row_lo), 0));
                cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d_row_hi), 0));
                mm &= ~1ull;
            }
            auto open_at = [&](int first) {
                asm volatile("" : "+s"(first));
                cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d_row_lo), first));
                cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d_row_hi), first));
                macc = mfma_acc{0.f, 0.f, 0.f, 0.f};
            };
            for (int g0 = 0; g0 < ngroups; g0 += 4) {
                float av[4], bv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    av[u] = pm[(g0 + u) * 48];
                    bv[u] = pm[(g0 + u) * 48 + 8];
                }
                const unsigned m16 = static_cast<unsigned>(mm) & 0xffffu;
                mm >>= 16;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (g0 + u < ngroups) {
                        const unsigned m4 = (m16 >> (4 * u)) & 5u;
                        if (__builtin_expect(m4 != 0u, 0)) {
                            if (m4 & 1u) {
                                flush_matrix();
                                open_at(4 * (g0 + u));
                            }
                            if (m4 & 4u) {
                                macc = __builtin_amdgcn_mfma_f32_16x16x4f32(lane < 32 ? av[u] : 0.f, bv[u], macc, 0, 0, 0);
                                flush_matrix();
                                open_at(4 * (g0 + u) + 2);
                                macc = __builtin_amdgcn_mfma_f32_16x16x4f32(lane < 32 ? 0.f : av[u], bv[u], macc, 0, 0, 0);
                            } else {
                                macc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], bv[u], macc, 0, 0, 0);
                            }
                        } else {
                            macc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], bv[u], macc, 0, 0, 0);
                        }
                    }
                }
            }
            wave_lds_fence();
            continue;
        }

        // Phase 2 is a chain of short dependent steps (a test, a branch, one multiply-add), bound by their latency, where
        // phase 1 is vector arithmetic: a wavefront in phase 2 goes first when both are ready (1.5 % of the kernel).
        __builtin_amdgcn_s_setprio(1);
        // phase 2: lane = (half, theta_t, Rs_s); the halves take alternate records.  Records past
        // `total` in the last step are zeros, so whole groups of eight pairs can always be run.
        const int npairs = min(64, total - base) >> 1;
        const T* pa = &S.rec[L.half][ang_t];
        const T* pg = &S.rec[L.half][8 + ang_s];
        const T* pda = pa;
        const T* ph = pg;
        if constexpr (kJvp) {
            pda = &S.jvp.rec2[L.half][ang_t];
            ph = &S.jvp.rec2[L.half][8 + ang_s];
        }
        // float: the four lanes of a quad (same theta_t) each read A_t of one of four consecutive pairs, and the
        // product takes it from the quad lane that holds it: one LDS read of A (and of dA_t) serves four pairs
        constexpr bool kQuadA = sizeof(T) == 4;
        const T* pa4 = &S.rec[L.half + 2 * ang_s][ang_t];
        const T* pda4 = pa4;
        if constexpr (kJvp) pda4 = &S.jvp.rec2[L.half + 2 * ang_s][ang_t];
        unsigned long long mm = starts;
        if (base == 0) {            // the batch's first segment opens here; nothing to close
            cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d_row_lo), 0));
            cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d_row_hi), 0));
            mm &= ~1ull;
        }
        struct Group {
            T a[kQuadA ? 2 : 8], g[8], da[!kJvp ? 1 : kQuadA ? 2 : 8], h[kJvp ? 8 : 1];
        };
        auto load8 = [&](int q0, Group& v) {
            if constexpr (kQuadA) {
                v.a[0] = pa4[q0 * 24];
                v.a[1] = pa4[(q0 + 4) * 24];
                if constexpr (kJvp) {
                    v.da[0] = pda4[q0 * 24];
                    v.da[1] = pda4[(q0 + 4) * 24];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if constexpr (!kQuadA) v.a[u] = pa[(q0 + u) * 24];
                v.g[u] = pg[(q0 + u) * 24];
                if constexpr (kJvp) {
                    if constexpr (!kQuadA) v.da[u] = pda[(q0 + u) * 24];
                    v.h[u] = ph[(q0 + u) * 24];
                }
            }
        };
        auto run8 = [&](int q0, const Group& v) {
            const unsigned m16 = static_cast<unsigned>(mm) & 0xffffu;     // this group's 16 slots
            mm >>= 16;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (__builtin_expect((m16 >> (2 * u)) & 1u, 0)) {
                    // a segment starts at record pair q0+u: close the open one, open the new one
                    flush();
                    int first = 2 * (q0 + u);
                    asm volatile("" : "+s"(first));      // keeps the lane reads inside this branch
                    cur_lo = static_cast<unsigned>(lane_read(static_cast<int>(d_row_lo), first));
                    cur_hi = static_cast<unsigned>(lane_read(static_cast<int>(d_row_hi), first));
                    acc = T(0);
                }
                if constexpr (kJvp && kQuadA) acc = fma_quad(v.da[u >> 2], u & 3, v.g[u], fma_quad(v.a[u >> 2], u & 3, v.h[u], acc));
                else if constexpr (kJvp) acc = fma(v.da[u], v.g[u], fma(v.a[u], v.h[u], acc));
                else if constexpr (kQuadA) acc = fma_quad(v.a[u >> 2], u & 3, v.g[u], acc);
                else acc = fma(v.a[u], v.g[u], acc);
            }
        };
        // eight record pairs per group, the next group's LDS reads in flight while one is summed
        Group v0, v1;
        load8(0, v0);
        for (int q0 = 0; q0 < npairs; q0 += 16) {
            const bool more1 = q0 + 8 < npairs;
            if (more1) load8(q0 + 8, v1);
            run8(q0, v0);
            if (more1) {
                if (q0 + 16 < npairs) load8(q0 + 16, v0);
                run8(q0 + 8, v1);
            }
        }
        __builtin_amdgcn_s_setprio(0);
        wave_lds_fence();
    }
    if (total > 0) {
        if constexpr (kMatrixPhase2) flush_matrix();
        else flush();
    }

    // ------------------------------------------------ segments without triples are zeros
    // The rows' addresses of the batch's empty segments are compacted into the (now free) table of row addresses, and
    // the lanes clear them a line at a time: a segment's 32 values are 128 (float) or 256 (double) consecutive bytes,
    // taken by 8 or 16 lanes with one 16-byte store each, so that one instruction writes 8 (4) whole segments and the
    // memory system sees full lines.  (One segment per lane, eight 16-byte stores each, is the same bytes in eight
    // times the write transactions, each a sixth of a line.)  Rows that are not 16-byte aligned: 4-byte stores.
    {
        const bool is_empty = lane < nb * kNumPairBlocks && cnt == 0;
        const unsigned long long empties = wave_ballot(is_empty);
        if (empties) {
            const bool unaligned = wave_ballot(is_empty && (seg_row_lo & 15u) != 0u) != 0ull;
            if (!unaligned) {
                constexpr int kLanesPer = kAngBlock * static_cast<int>(sizeof(T)) / 16;      // lanes per segment: 8 or 16
                constexpr int kPerStep = 64 / kLanesPer;
                const int n_empty = popc64(empties);
                if (is_empty) S.segrow[popc64(empties & lt_mask)] = (static_cast<unsigned long long>(seg_row_hi) << 32) | seg_row_lo;
                wave_lds_fence();
                for (int e0 = 0; e0 < n_empty; e0 += kPerStep) {
                    const int e = e0 + lane / kLanesPer;
                    if (e < n_empty) {
                        char* dst = reinterpret_cast<char*>(S.segrow[e]) + (lane % kLanesPer) * 16;
                        store_global16(dst);
                    }
                }
                wave_lds_fence();
            } else if (is_empty) {
                T* dst = reinterpret_cast<T*>((static_cast<unsigned long long>(seg_row_hi) << 32) | seg_row_lo);
                for (int q = 0; q < kAngBlock; ++q) store_global(dst + q, T(0));
            }
        }
    }
}

}  // namespace khan
