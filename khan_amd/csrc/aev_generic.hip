// General-shape AEV forward and backward kernels for gfx950.
//
// These accept any molecule size and any neighbour count: one workgroup of four wavefronts per
// molecule, one wavefront per centre atom at a time.  Partner atoms are scanned 64 at a time (one
// per lane); lanes inside a cutoff are found with a ballot and visited by broadcasting their data,
// so nothing has to fit a fixed-size neighbour list.  While a centre is processed the 64 lanes hold
// the centre's output row itself:
//     radial  lane = (partner type, shell)        64 slots = 4 types x 16 shells
//     angular lane = (half, theta_t, Rs_s)        2 halves x 32 slots; the halves take alternate k
// so a centre's 384-wide row is accumulated by its own wavefront and stored once, coalesced, with no
// global atomics (forward).  The backward pass recomputes the geometry, reduces the three weighted
// sums of each triple across the 32 (t,s) lanes, and adds forces on j, k and i.
//
// Semantics follow the reference CPU kernels: forward gpu_featurizer/kernel_cpu.cpp:406-537,
// backward kernel_cpu.cpp:217-366 (strict < on both cutoffs, i != j != k, j < k, types other than
// 0,1,2 go to the O bucket).  cos(theta - theta_t) is evaluated as c cos(theta_t) + s sin(theta_t)
// with c from the dot product and s from the cross product, which avoids acos and stays accurate
// for nearly collinear triples.
#include "aev_generic_center.h"

namespace khan {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void zero3_kernel(T* a, T* b, T* c, int64_t n)
{
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g < n) {
        a[g] = T(0);
        b[g] = T(0);
        c[g] = T(0);
    }
}

// ------------------------------------------------------------------------------------ forward
template <typename T>
__global__ __launch_bounds__(256) void aev_fwd_generic_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, const int32_t* __restrict__ SIs, Buckets<T> out, int min_atoms)
{
    __shared__ T ang_rows[4][kAngular];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int mol = blockIdx.x;
    const int n = MACs[mol], off = MOs[mol];
    if (n < min_atoms) return;        // smaller molecules are handled by the small-molecule kernel
    const LaneConsts<T> L = lane_consts<T>(lane);
    T* ang = ang_rows[wave];

    for (int i = wave; i < n; i += 4) {
        T* row = out.p[fold_type(A[off + i])] + static_cast<size_t>(SIs[off + i]) * kFeats;
        fwd_center_generic<T>(L, lane, X, Y, Z, A, off, n, i, ang, row);
    }
}

// ----------------------------------------------------------------------------------- backward
template <typename T>
__global__ __launch_bounds__(256) void aev_bwd_generic_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, const int32_t* __restrict__ SIs, Buckets<const T> gin,
    T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ)
{
    __shared__ T g_rows[4][kAngular];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int mol = blockIdx.x;
    const int n = MACs[mol], off = MOs[mol];
    const LaneConsts<T> L = lane_consts<T>(lane);
    T* g_ang = g_rows[wave];

    for (int i = wave; i < n; i += 4) {
        const T* grow = gin.p[fold_type(A[off + i])] + static_cast<size_t>(SIs[off + i]) * kFeats;
        const T g_rad = grow[lane];                       // upstream for slot (rtype, shell)
        for (int q = lane; q < kAngular; q += 64) g_ang[q] = grow[kRadial + q];
        wave_lds_fence();
        const T xi = X[off + i], yi = Y[off + i], zi = Z[off + i];
        T ix = T(0), iy = T(0), iz = T(0);   // gradient on i: per-half partials, summed at the end

        for (int jc = 0; jc < n; jc += 64) {
            const int j = jc + lane;
            const Partner<T> pj = scan_partner(X, Y, Z, A, off, j, n, xi, yi, zi);
            const bool valid = (j < n) && (j != i);
            const bool inR = valid && (pj.r < L.R_Rc);
            const bool inA = valid && (pj.r < L.A_Rc);
            const T fcR = inR ? cutoff_fn(pj.r, L.pi_rc_R) : T(0);
            const T dfcR = inR ? cutoff_dfn(pj.r, L.pi_rc_R) : T(0);
            const T fcA = inA ? cutoff_fn(pj.r, L.pi_rc_A) : T(0);
            const T dfcA = inA ? cutoff_dfn(pj.r, L.pi_rc_A) : T(0);

            // radial: dE/dr_ij = sum_shells g * exp(-eta d^2) * (f_C' - 2 eta d f_C)
            for (unsigned long long m = wave_ballot(inR); m; m &= m - 1) {
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
                    atomicAdd(&gX[off + jc + b], -fx);
                    atomicAdd(&gY[off + jc + b], -fy);
                    atomicAdd(&gZ[off + jc + b], -fz);
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
                        kin = (k < n) && (k != i) && (pk.r < L.A_Rc);
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
                        // guard: exactly collinear triples have no finite derivative
                        const T s = fmax(Real<T>::sqrt_(cx * cx + cy * cy + cz * cz), T(1e-30));
                        const T base = T(1) + c * L.ct + s * L.st;
                        const T b2 = base * base, b4 = b2 * b2;
                        const T Am1 = b4 * b2 * base;                         // base^(zeta-1)
                        const T At = Am1 * base;
                        const T dAt = T(8) * Am1 * (L.ct - (c / s) * L.st);   // d/dc (1+cos(th-th_t))^8
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
                                atomicAdd(&gX[off + kc + src], -vkx);
                                atomicAdd(&gY[off + kc + src], -vky);
                                atomicAdd(&gZ[off + kc + src], -vkz);
                            }
                        }
                    }
                }
                jx += __shfl_xor(jx, 32, 64);
                jy += __shfl_xor(jy, 32, 64);
                jz += __shfl_xor(jz, 32, 64);
                if (lane == 0) {
                    atomicAdd(&gX[off + jc + bj], -jx);
                    atomicAdd(&gY[off + jc + bj], -jy);
                    atomicAdd(&gZ[off + jc + bj], -jz);
                }
            }
        }
        ix += __shfl_xor(ix, 32, 64);
        iy += __shfl_xor(iy, 32, 64);
        iz += __shfl_xor(iz, 32, 64);
        if (lane == 0) {
            atomicAdd(&gX[off + i], ix);
            atomicAdd(&gY[off + i], iy);
            atomicAdd(&gZ[off + i], iz);
        }
        wave_lds_fence();
    }
}

}  // namespace

template <typename T>
hipError_t launch_fwd_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, Buckets<T> out, int min_atoms, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    aev_fwd_generic_kernel<T><<<dim3(n_mols), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, SIs, out, min_atoms);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_bwd_generic(const T* X, const T* Y, const T* Z, const int32_t* A,
                              const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                              const int32_t* SIs, Buckets<const T> g, T* gX, T* gY, T* gZ,
                              int64_t n_atoms, hipStream_t stream)
{
    // outputs are accumulated with atomics, so they start from zero (functor_op_cpu.cpp:70-72);
    // a fill kernel rather than a memset node keeps the sequence safe to capture in a HIP graph
    if (n_atoms > 0) {
        const int64_t blocks = (n_atoms + 255) / 256;
        zero3_kernel<T><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(gX, gY, gZ, n_atoms);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (n_mols <= 0) return hipSuccess;
    aev_bwd_generic_kernel<T><<<dim3(n_mols), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, SIs, g, gX, gY, gZ);
    return hipGetLastError();
}

template hipError_t launch_fwd_generic<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<float>, int, hipStream_t);
template hipError_t launch_fwd_generic<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<double>, int, hipStream_t);
template hipError_t launch_bwd_generic<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const float>, float*, float*, float*, int64_t, hipStream_t);
template hipError_t launch_bwd_generic<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const double>, double*, double*, double*, int64_t, hipStream_t);

}  // namespace khan
