// Per-centre building blocks of the general-shape AEV kernels, shared by the general kernel and by
// the small-molecule kernel (which falls back to them for centres that overflow its neighbour lists).
#pragma once
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

template <typename T>
struct LaneConsts {
    T ct, st, ars;        // angular: cos/sin(theta_t), Rs_s of this lane's (t,s) slot
    T rrs;                // radial: Rs of this lane's shell
    int rtype;            // radial: partner type of this lane's slot
    int ts, half;
    T pi_rc_R, pi_rc_A, R_Rc, A_Rc, R_eta, A_eta;
};

template <typename T>
__device__ __forceinline__ LaneConsts<T> lane_consts(int lane)
{
    LaneConsts<T> c;
    c.ts = lane & 31;
    c.half = lane >> 5;
    const int t = c.ts >> 2, s = c.ts & 3;
    c.ct = static_cast<T>(kCosTheta[t]);
    c.st = static_cast<T>(kSinTheta[t]);
    c.ars = static_cast<T>(kA_Rs_f[s]);
    c.rrs = static_cast<T>(kR_Rs_f[lane & 15]);
    c.rtype = lane >> 4;
    c.R_Rc = static_cast<T>(kR_Rc_f);
    c.A_Rc = static_cast<T>(kA_Rc_f);
    c.R_eta = static_cast<T>(kR_eta_f);
    c.A_eta = static_cast<T>(kA_eta_f);
    c.pi_rc_R = static_cast<T>(kPi / static_cast<double>(kR_Rc_f));
    c.pi_rc_A = static_cast<T>(kPi / static_cast<double>(kA_Rc_f));
    return c;
}

// data of one scanned partner atom, held by the lane that scanned it
template <typename T>
struct Partner {
    T dx, dy, dz, r;
    int type;
};

template <typename T>
__device__ __forceinline__ Partner<T> scan_partner(const T* X, const T* Y, const T* Z,
                                                   const int32_t* A, int off, int j, int n, T xi,
                                                   T yi, T zi)
{
    Partner<T> p;
    p.dx = p.dy = p.dz = T(0);
    p.r = T(1e30);
    p.type = 0;
    if (j < n) {
        p.dx = xi - X[off + j];
        p.dy = yi - Y[off + j];
        p.dz = zi - Z[off + j];
        p.r = Real<T>::sqrt_(p.dx * p.dx + p.dy * p.dy + p.dz * p.dz);
        p.type = fold_type(A[off + j]);
    }
    return p;
}

template <typename T>
__device__ __forceinline__ Partner<T> partner_from_lane(const Partner<T>& p, int src)
{
    Partner<T> q;
    q.dx = wave_get(p.dx, src);
    q.dy = wave_get(p.dy, src);
    q.dz = wave_get(p.dz, src);
    q.r = wave_get(p.r, src);
    q.type = wave_get(p.type, src);
    return q;
}

// Adds `val` to slot (blk, ts) of a centre's angular row in LDS.  The two half-waves hold two different
// triples; their 32 slots collide only when both triples fall into the same type-pair block, in which case
// the lower half adds both values.  A plain read-add-write then touches distinct addresses across the wave
// (float atomics on LDS cost two orders of magnitude more per wave instruction on this part).
template <typename T>
__device__ __forceinline__ void ang_accumulate(T* ang, int blk, int ts, int half, bool act, T val)
{
    const T v = act ? val : T(0);
    const int mine = act ? blk : -1;
    const int other = __shfl_xor(mine, 32, 64);
    const T other_v = __shfl_xor(v, 32, 64);
    const bool same = mine == other;
    if (act && (!same || half == 0)) ang[blk * kAngBlock + ts] += same ? v + other_v : v;
}

// Forward pass of ONE centre atom i of the molecule at [off, off+n), executed by one whole wavefront.
// `ang` is kAngular elements of this wavefront's LDS; the finished 384-wide row is stored to `row`.
template <typename T>
__device__ __forceinline__ void fwd_center_generic(const LaneConsts<T>& L, int lane, const T* __restrict__ X,
                                                   const T* __restrict__ Y, const T* __restrict__ Z,
                                                   const int32_t* __restrict__ A, int off, int n, int i,
                                                   T* ang, T* __restrict__ row)
{
        for (int q = lane; q < kAngular; q += 64) ang[q] = T(0);
        wave_lds_fence();
        const T xi = X[off + i], yi = Y[off + i], zi = Z[off + i];
        T acc_rad = T(0);

        for (int jc = 0; jc < n; jc += 64) {
            const int j = jc + lane;
            const Partner<T> pj = scan_partner(X, Y, Z, A, off, j, n, xi, yi, zi);
            const bool valid = (j < n) && (j != i);
            const bool inR = valid && (pj.r < L.R_Rc);
            const bool inA = valid && (pj.r < L.A_Rc);
            const T fcR = inR ? cutoff_fn(pj.r, L.pi_rc_R) : T(0);
            const T fcA = inA ? cutoff_fn(pj.r, L.pi_rc_A) : T(0);

            // radial: every partner inside R_Rc adds 16 shell values to the slots of its type
            for (unsigned long long m = wave_ballot(inR); m; m &= m - 1) {
                const int b = lowest_bit(m);
                const T rb = wave_get(pj.r, b), fb = wave_get(fcR, b);
                const int tb = wave_get(pj.type, b);
                const T d = rb - L.rrs;
                const T g = Real<T>::exp_(-L.R_eta * d * d) * fb;
                acc_rad += (tb == L.rtype) ? g : T(0);
            }

            // angular: j from this chunk, k > j from this and later chunks
            for (unsigned long long mj = wave_ballot(inA); mj; mj &= mj - 1) {
                const int bj = lowest_bit(mj);
                const Partner<T> J = partner_from_lane(pj, bj);
                const T Jfc = wave_get(fcA, bj);
                for (int kc = jc; kc < n; kc += 64) {
                    Partner<T> pk;
                    T fcK;
                    bool kin;
                    if (kc == jc) {
                        pk = pj;
                        fcK = fcA;
                        kin = inA && (lane > bj);
                    } else {
                        const int k = kc + lane;
                        pk = scan_partner(X, Y, Z, A, off, k, n, xi, yi, zi);
                        kin = (k < n) && (k != i) && (pk.r < L.A_Rc);
                        fcK = kin ? cutoff_fn(pk.r, L.pi_rc_A) : T(0);
                    }
                    unsigned long long mk = wave_ballot(kin);
                    while (mk) {
                        const int b0 = lowest_bit(mk);
                        mk &= mk - 1;
                        int b1 = -1;
                        if (mk) {
                            b1 = lowest_bit(mk);
                            mk &= mk - 1;
                        }
                        const bool act = (L.half == 0) || (b1 >= 0);
                        const int src = (L.half == 0 || b1 < 0) ? b0 : b1;
                        const Partner<T> K = partner_from_lane(pk, src);
                        const T Kfc = wave_get(fcK, src);

                        const T inv = T(1) / (J.r * K.r);
                        T c = (J.dx * K.dx + J.dy * K.dy + J.dz * K.dz) * inv;
                        c = fmin(fmax(c, T(-1)), T(1));
                        const T cx = J.dy * K.dz - J.dz * K.dy;
                        const T cy = J.dz * K.dx - J.dx * K.dz;
                        const T cz = J.dx * K.dy - J.dy * K.dx;
                        // (a coincident partner makes c and s 0/0: the clamps turn them into -1 and 0, the angle pi the
                        // reference arrives at through fmax/fmin/acos, kernel_cpu.cpp:514-517)
                        const T s = fmin(fmax(Real<T>::sqrt_(cx * cx + cy * cy + cz * cz) * inv, T(0)), T(1));
                        const T base = T(1) + c * L.ct + s * L.st;
                        const T b2 = base * base, b4 = b2 * b2, b8 = b4 * b4;
                        const T dav = (J.r + K.r) * T(0.5) - L.ars;
                        const T val = T(0.0078125) * b8 * Real<T>::exp_(-L.A_eta * dav * dav) * Jfc * Kfc;
                        ang_accumulate(ang, pair_block(J.type, K.type), L.ts, L.half, act, val);
                    }
                }
            }
        }

        wave_lds_fence();
        row[lane] = acc_rad;
        for (int q = lane; q < kAngular; q += 64) row[kRadial + q] = ang[q];
        wave_lds_fence();
}

// Backward pass of ONE centre atom i (general shape), executed by one whole wavefront: adds
// dL/dxyz of every atom touched by centre i's row through `add(atom, fx, fy, fz)`, where `atom` is
// the index inside the molecule.  `g_ang` is kAngular elements of this wavefront's LDS and `grow` the
// centre's upstream 384-wide row.  Reference: kernel_cpu.cpp:217-366.
template <typename T, typename AddForce>
__device__ __forceinline__ void bwd_center_generic(const LaneConsts<T>& L, int lane, const T* __restrict__ X,
                                                   const T* __restrict__ Y, const T* __restrict__ Z,
                                                   const int32_t* __restrict__ A, int off, int n, int i,
                                                   T* g_ang, const T* __restrict__ grow, AddForce add,
                                                   bool with_radial = true)
{
        const T g_rad = grow[lane];                       // upstream for slot (rtype, shell)
        for (int q = lane; q < kAngular; q += 64) g_ang[q] = grow[kRadial + q];
        wave_lds_fence();
        const T xi = X[off + i], yi = Y[off + i], zi = Z[off + i];
        T ix = T(0), iy = T(0), iz = T(0);   // gradient on i: per-half partials, summed at the end

        for (int jc = 0; jc < n; jc += 64) {
            const int j = jc + lane;
            const Partner<T> pj = scan_partner(X, Y, Z, A, off, j, n, xi, yi, zi);
            const bool valid = (j < n) && (j != i);
            const bool inR = valid && (pj.r < L.R_Rc) && (pj.r > T(0));      // no derivative for a coincident atom
            const bool inA = valid && (pj.r < L.A_Rc) && (pj.r > T(0));
            const T fcR = inR ? cutoff_fn(pj.r, L.pi_rc_R) : T(0);
            const T dfcR = inR ? cutoff_dfn(pj.r, L.pi_rc_R) : T(0);
            const T fcA = inA ? cutoff_fn(pj.r, L.pi_rc_A) : T(0);
            const T dfcA = inA ? cutoff_dfn(pj.r, L.pi_rc_A) : T(0);

            // radial: dE/dr_ij = sum_shells g * exp(-eta d^2) * (f_C' - 2 eta d f_C)
            // (a caller that has already done the centre's radial pairs passes with_radial = false)
            for (unsigned long long m = with_radial ? wave_ballot(inR) : 0ull; m; m &= m - 1) {
                const int b = lowest_bit(m);
                const Partner<T> J = partner_from_lane(pj, b);
                const T fb = wave_get(fcR, b), dfb = wave_get(dfcR, b);
                const T d = J.r - L.rrs;
                T w = g_rad * Real<T>::exp_(-L.R_eta * d * d) * (dfb - T(2) * L.R_eta * d * fb);
                w = (J.type == L.rtype) ? w : T(0);
                const T G = wave_sum(w) / J.r;            // dE/dr divided by r: multiplies d = x_i - x_j
                const T fx = G * J.dx, fy = G * J.dy, fz = G * J.dz;
                if (L.half == 0) { ix += fx; iy += fy; iz += fz; }
                if (lane == 0) {
                    add(jc + b, -fx, -fy, -fz);
                }
            }

            // angular
            for (unsigned long long mj = wave_ballot(inA); mj; mj &= mj - 1) {
                const int bj = lowest_bit(mj);
                const Partner<T> J = partner_from_lane(pj, bj);
                const T Jfc = wave_get(fcA, bj), Jdfc = wave_get(dfcA, bj);
                const T Jinv = T(1) / J.r;
                const T ujx = J.dx * Jinv, ujy = J.dy * Jinv, ujz = J.dz * Jinv;
                T jx = T(0), jy = T(0), jz = T(0);          // force on j: per-half partials
                for (int kc = jc; kc < n; kc += 64) {
                    Partner<T> pk;
                    T fcK, dfcK;
                    bool kin;
                    if (kc == jc) {
                        pk = pj;
                        fcK = fcA;
                        dfcK = dfcA;
                        kin = inA && (lane > bj);
                    } else {
                        const int k = kc + lane;
                        pk = scan_partner(X, Y, Z, A, off, k, n, xi, yi, zi);
                        kin = (k < n) && (k != i) && (pk.r < L.A_Rc) && (pk.r > T(0));
                        fcK = kin ? cutoff_fn(pk.r, L.pi_rc_A) : T(0);
                        dfcK = kin ? cutoff_dfn(pk.r, L.pi_rc_A) : T(0);
                    }
                    unsigned long long mk = wave_ballot(kin);
                    while (mk) {
                        const int b0 = lowest_bit(mk);
                        mk &= mk - 1;
                        int b1 = -1;
                        if (mk) {
                            b1 = lowest_bit(mk);
                            mk &= mk - 1;
                        }
                        const bool act = (L.half == 0) || (b1 >= 0);
                        const int src = (L.half == 0 || b1 < 0) ? b0 : b1;
                        const Partner<T> K = partner_from_lane(pk, src);
                        const T Kfc = wave_get(fcK, src), Kdfc = wave_get(dfcK, src);
                        const T Kinv = T(1) / K.r;
                        const T ukx = K.dx * Kinv, uky = K.dy * Kinv, ukz = K.dz * Kinv;

                        T c = ujx * ukx + ujy * uky + ujz * ukz;
                        c = fmin(fmax(c, T(-1)), T(1));
                        const T cx = ujy * ukz - ujz * uky;
                        const T cy = ujz * ukx - ujx * ukz;
                        const T cz = ujx * uky - ujy * ukx;
                        const T s = Real<T>::sqrt_(cx * cx + cy * cy + cz * cz);
                        const T base = T(1) + c * L.ct + s * L.st;
                        const T b2 = base * base, b4 = b2 * b2;
                        const T Am1 = b4 * b2 * base;                         // base^(zeta-1)
                        const T At = Am1 * base;
                        const T dAt = T(8) * Am1 * (L.ct - cot_reg(c, s) * L.st);   // d/dc (1+cos(th-th_t))^8; zero cot on the line
                        const T dav = (J.r + K.r) * T(0.5) - L.ars;
                        const T Gs = Real<T>::exp_(-L.A_eta * dav * dav);
                        const T g = g_ang[pair_block(J.type, K.type) * kAngBlock + L.ts];
                        const T gAG = g * At * Gs;
                        const T W0 = half_sum(gAG);
                        const T Wc = half_sum(g * dAt * Gs);
                        const T Wr = half_sum(gAG * (T(-2) * L.A_eta * dav));

                        const T two_pow = T(0.0078125);
                        const T P = two_pow * Jfc * Kfc;
                        const T Fj = P * Wr * T(0.5) + two_pow * W0 * Jdfc * Kfc;   // dE/dr_ij
                        const T Fk = P * Wr * T(0.5) + two_pow * W0 * Jfc * Kdfc;   // dE/dr_ik
                        const T Fc = P * Wc;                                        // dE/dcos
                        const T vjx = Fj * ujx + Fc * (ukx - c * ujx) * Jinv;
                        const T vjy = Fj * ujy + Fc * (uky - c * ujy) * Jinv;
                        const T vjz = Fj * ujz + Fc * (ukz - c * ujz) * Jinv;
                        const T vkx = Fk * ukx + Fc * (ujx - c * ukx) * Kinv;
                        const T vky = Fk * uky + Fc * (ujy - c * uky) * Kinv;
                        const T vkz = Fk * ukz + Fc * (ujz - c * ukz) * Kinv;
                        if (act) {
                            ix += vjx + vkx; iy += vjy + vky; iz += vjz + vkz;
                            jx += vjx; jy += vjy; jz += vjz;
                            if (L.ts == 0) {
                                add(kc + src, -vkx, -vky, -vkz);
                            }
                        }
                    }
                }
                jx += __shfl_xor(jx, 32, 64);
                jy += __shfl_xor(jy, 32, 64);
                jz += __shfl_xor(jz, 32, 64);
                if (lane == 0) {
                    add(jc + bj, -jx, -jy, -jz);
                }
            }
        }
        ix += __shfl_xor(ix, 32, 64);
        iy += __shfl_xor(iy, 32, 64);
        iz += __shfl_xor(iz, 32, 64);
        if (lane == 0) {
            add(i, ix, iy, iz);
        }
        wave_lds_fence();
}

// Jacobian-vector product of ONE centre atom i (general shape), executed by one whole wavefront:
// row[f] = sum_a dAEV_i[f]/dx_a . v_a with v_a = (VX[a], VY[a], VZ[a]), a = i and its partners.
// Lanes hold the output slots as in the forward routine; every term of the forward sum is replaced
// by its derivative along v:  d r_ij = u_ij.(v_i - v_j),  d cos = ((u_k - c u_j).w_j)/r_j +
// ((u_j - c u_k).w_k)/r_k.  `ang` is kAngular elements of this wavefront's LDS.
// Contraction of the reference's featurize_grad_inverse (kernel_cpu.cpp:37-179), with the incoming
// vectors read by atom index.
template <typename T>
__device__ __forceinline__ void jvp_center_generic(const LaneConsts<T>& L, int lane, const T* __restrict__ X,
                                                   const T* __restrict__ Y, const T* __restrict__ Z,
                                                   const int32_t* __restrict__ A,
                                                   const T* __restrict__ VX, const T* __restrict__ VY,
                                                   const T* __restrict__ VZ, int off, int n, int i,
                                                   T* ang, T* __restrict__ row)
{
        for (int q = lane; q < kAngular; q += 64) ang[q] = T(0);
        wave_lds_fence();
        const T xi = X[off + i], yi = Y[off + i], zi = Z[off + i];
        const T vxi = VX[off + i], vyi = VY[off + i], vzi = VZ[off + i];
        T acc_rad = T(0);

        // a scanned partner plus what the derivative needs: relative vector w = v_i - v_j, d r = u.w
        struct Extra {
            T wx, wy, wz, rd;
        };
        auto scan_extra = [&](const Partner<T>& p, int j) {
            Extra e;
            e.wx = e.wy = e.wz = e.rd = T(0);
            if (j < n && p.r > T(0)) {
                e.wx = vxi - VX[off + j];
                e.wy = vyi - VY[off + j];
                e.wz = vzi - VZ[off + j];
                e.rd = (p.dx * e.wx + p.dy * e.wy + p.dz * e.wz) / p.r;
            }
            return e;
        };
        auto extra_from_lane = [&](const Extra& e, int src) {
            Extra q;
            q.wx = wave_get(e.wx, src);
            q.wy = wave_get(e.wy, src);
            q.wz = wave_get(e.wz, src);
            q.rd = wave_get(e.rd, src);
            return q;
        };

        for (int jc = 0; jc < n; jc += 64) {
            const int j = jc + lane;
            const Partner<T> pj = scan_partner(X, Y, Z, A, off, j, n, xi, yi, zi);
            const Extra ej = scan_extra(pj, j);
            const bool valid = (j < n) && (j != i);
            const bool inR = valid && (pj.r < L.R_Rc) && (pj.r > T(0));      // no derivative for a coincident atom
            const bool inA = valid && (pj.r < L.A_Rc) && (pj.r > T(0));
            const T fcR = inR ? cutoff_fn(pj.r, L.pi_rc_R) : T(0);
            const T dfcR = inR ? cutoff_dfn(pj.r, L.pi_rc_R) : T(0);
            const T fcA = inA ? cutoff_fn(pj.r, L.pi_rc_A) : T(0);
            const T dfcA = inA ? cutoff_dfn(pj.r, L.pi_rc_A) : T(0);

            // radial: d/dr [exp(-eta d^2) f_C] * d r
            for (unsigned long long m = wave_ballot(inR); m; m &= m - 1) {
                const int b = lowest_bit(m);
                const T rb = wave_get(pj.r, b), fb = wave_get(fcR, b), dfb = wave_get(dfcR, b);
                const T rdb = wave_get(ej.rd, b);
                const int tb = wave_get(pj.type, b);
                const T d = rb - L.rrs;
                const T g = Real<T>::exp_(-L.R_eta * d * d) * (dfb - T(2) * L.R_eta * d * fb) * rdb;
                acc_rad += (tb == L.rtype) ? g : T(0);
            }

            // angular: j from this chunk, k > j from this and later chunks
            for (unsigned long long mj = wave_ballot(inA); mj; mj &= mj - 1) {
                const int bj = lowest_bit(mj);
                const Partner<T> J = partner_from_lane(pj, bj);
                const Extra Je = extra_from_lane(ej, bj);
                const T Jfc = wave_get(fcA, bj), Jdfc = wave_get(dfcA, bj);
                const T Jinv = T(1) / J.r;
                const T ujx = J.dx * Jinv, ujy = J.dy * Jinv, ujz = J.dz * Jinv;
                for (int kc = jc; kc < n; kc += 64) {
                    Partner<T> pk;
                    Extra ek;
                    T fcK, dfcK;
                    bool kin;
                    if (kc == jc) {
                        pk = pj;
                        ek = ej;
                        fcK = fcA;
                        dfcK = dfcA;
                        kin = inA && (lane > bj);
                    } else {
                        const int k = kc + lane;
                        pk = scan_partner(X, Y, Z, A, off, k, n, xi, yi, zi);
                        ek = scan_extra(pk, k);
                        kin = (k < n) && (k != i) && (pk.r < L.A_Rc) && (pk.r > T(0));
                        fcK = kin ? cutoff_fn(pk.r, L.pi_rc_A) : T(0);
                        dfcK = kin ? cutoff_dfn(pk.r, L.pi_rc_A) : T(0);
                    }
                    unsigned long long mk = wave_ballot(kin);
                    while (mk) {
                        const int b0 = lowest_bit(mk);
                        mk &= mk - 1;
                        int b1 = -1;
                        if (mk) {
                            b1 = lowest_bit(mk);
                            mk &= mk - 1;
                        }
                        const bool act = (L.half == 0) || (b1 >= 0);
                        const int src = (L.half == 0 || b1 < 0) ? b0 : b1;
                        const Partner<T> K = partner_from_lane(pk, src);
                        const Extra Ke = extra_from_lane(ek, src);
                        const T Kfc = wave_get(fcK, src), Kdfc = wave_get(dfcK, src);
                        const T Kinv = T(1) / K.r;
                        const T ukx = K.dx * Kinv, uky = K.dy * Kinv, ukz = K.dz * Kinv;

                        T c = ujx * ukx + ujy * uky + ujz * ukz;
                        c = fmin(fmax(c, T(-1)), T(1));
                        const T cx = ujy * ukz - ujz * uky;
                        const T cy = ujz * ukx - ujx * ukz;
                        const T cz = ujx * uky - ujy * ukx;
                        const T s = Real<T>::sqrt_(cx * cx + cy * cy + cz * cz);
                        const T dc = ((ukx - c * ujx) * Je.wx + (uky - c * ujy) * Je.wy + (ukz - c * ujz) * Je.wz) * Jinv +
                                     ((ujx - c * ukx) * Ke.wx + (ujy - c * uky) * Ke.wy + (ujz - c * ukz) * Ke.wz) * Kinv;
                        const T base = T(1) + c * L.ct + s * L.st;
                        const T b2 = base * base, b4 = b2 * b2;
                        const T Am1 = b4 * b2 * base;
                        const T At = Am1 * base;
                        const T dAt = T(8) * Am1 * (L.ct - cot_reg(c, s) * L.st) * dc;
                        const T dav = (J.r + K.r) * T(0.5) - L.ars;
                        const T Gs = Real<T>::exp_(-L.A_eta * dav * dav);
                        const T dGs = Gs * (T(-2) * L.A_eta * dav) * T(0.5) * (Je.rd + Ke.rd);
                        const T two_pow = T(0.0078125);
                        const T P = two_pow * Jfc * Kfc;
                        const T dP = two_pow * (Jdfc * Je.rd * Kfc + Jfc * Kdfc * Ke.rd);
                        const T val = dAt * Gs * P + At * (dGs * P + Gs * dP);
                        ang_accumulate(ang, pair_block(J.type, K.type), L.ts, L.half, act, val);
                    }
                }
            }
        }

        wave_lds_fence();
        row[lane] = acc_rad;
        for (int q = lane; q < kAngular; q += 64) row[kRadial + q] = ang[q];
        wave_lds_fence();
}

}  // namespace khan
