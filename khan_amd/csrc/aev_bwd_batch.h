// Pieces of the one-wavefront AEV backward pass shared by the small-molecule kernels (one wavefront per
// molecule, float and double) and the medium-molecule kernel (four wavefronts per molecule): the pooled
// neighbour lists of a batch of centres, the radial pull of one (centre, partner) pair, the staging of the
// upstream rows, and the round-robin angular walk.
#pragma once
#include "aev_small_common.h"

namespace khan {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f* global_v4f_ptr;    // a 16-byte piece of a row in HBM

constexpr int kBlockStride = 36;   // elements between staged 32-element blocks: rotates the LDS banks

// per-wavefront LDS of a batch: the centres' angular partner lists laid end to end (at most 64 entries)
// and their rows' angular upstream values
template <typename T, int kNB = kB>
struct __align__(16) BwdPool {
    static constexpr int kCentres = kNB;          // centres per batch
    typename Fast<T>::vec4 nbr[64];               // unit vector (centre minus partner)/r, and r
    typename Fast<T>::vec4 facc[64];              // force on each list entry from its centre's row
    typename Fast<T>::vec2 nbr_fc[64];            // f_C(r, A_Rc) and its derivative in r
    T gst[kNB * kNumPairBlocks * kBlockStride];   // staged upstream blocks [centre][type pair][32]
    unsigned char nbr_idx[64];                    // sorted position of the partner
};

__device__ __forceinline__ int sel6(int b, int v0, int v1, int v2, int v3, int v4, int v5)
{
    return b == 0 ? v0 : b == 1 ? v1 : b == 2 ? v2 : b == 3 ? v3 : b == 4 ? v4 : v5;
}

// sum over the shells of g_q e_q (f_C' - 2 eta d_q f_C), e_q = exp(-eta d_q^2), d_q = r - Rs_q, for kN shells whose
// radii are rs[0..kN)
template <typename T, int kN>
__device__ __forceinline__ T radial_shell_sum(const T (&g)[kN], const T (&rs)[kN], T r, T fc, T dfc)
{
    const T m2eta_fc = T(-2) * static_cast<T>(kR_eta_f) * fc;
    T Gsum = T(0);
#pragma unroll
    for (int q = 0; q < kN; ++q) {
        const T d = r - rs[q];
        const T e = Fast<T>::gauss(static_cast<T>(kR_eta_f), d);
        Gsum = fma(g[q] * e, fma(m2eta_fc, d, dfc), Gsum);   // g e (f_C' - 2 eta d f_C)
    }
    return Gsum;
}

// Which shells a pair at distance r needs.  double: all 16.  float: the nine nearest to r -- a shell more than 4.5
// spacings (1.15 A) away contributes exp(-16 * 1.15^2) = 6e-10 times a factor that grows no faster than 2 eta d,
// in all less than 1e-8 of the largest term of the sum for every r below the cutoff: an order below the rounding of
// the float sum itself.  The window is [q0, q0 + 9) with q0 = clamp(nearest - 4, 0, 7).
template <typename T> struct ShellWindow {
    static constexpr int kShells = kNumRRs;
    static __device__ __forceinline__ int first(T) { return 0; }
};
template <> struct ShellWindow<float> {
    static constexpr int kShells = 9;
    static __device__ __forceinline__ int first(float r)
    {
        constexpr float kInvSpacing = 1.0f / 0.25625f;          // Rs_q = 0.5 + 0.25625 q
        const int nearest = __float2int_rn((r - 0.5f) * kInvSpacing);
        return min(max(nearest - 4, 0), kNumRRs - kShells);
    }
};

typedef float v4f_dword_aligned __attribute__((ext_vector_type(4), aligned(4)));
typedef const __attribute__((address_space(1))) v4f_dword_aligned* global_v4f_unaligned_ptr;
typedef const __attribute__((address_space(1))) float* global_float_ptr;

// the window's upstream values g[q0 .. q0 + kShells) of a 16-shell block, and the shells' radii
template <typename T>
__device__ __forceinline__ void load_shell_window(const T* block, int q0, T (&g)[ShellWindow<T>::kShells],
                                                  T (&rs)[ShellWindow<T>::kShells])
{
    if constexpr (sizeof(T) == 4) {
        // nine floats from a 4-byte-aligned address: two 16-byte loads and one of 4 bytes
        const global_v4f_unaligned_ptr gp = (global_v4f_unaligned_ptr)(block + q0);
        const v4f_dword_aligned a = gp[0], b = gp[1];
        g[0] = a.x; g[1] = a.y; g[2] = a.z; g[3] = a.w;
        g[4] = b.x; g[5] = b.y; g[6] = b.z; g[7] = b.w;
        g[8] = ((global_float_ptr)(block + q0))[8];
#pragma unroll
        for (int q = 0; q < 9; ++q) rs[q] = kR_Rs_f[q0 + q];
    } else {
        constexpr int kPieces = 16 * sizeof(T) / 16;          // 16-byte loads for the 16 upstream values
        union {
            v4f piece[kPieces];
            T gr[16];
        } u;
        const global_v4f_ptr gp = (global_v4f_ptr)block;
#pragma unroll
        for (int q = 0; q < kPieces; ++q) u.piece[q] = gp[q];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            g[q] = u.gr[q];
            rs[q] = static_cast<T>(kR_Rs_f[q]);
        }
    }
}

// Radial part of one (centre, partner) pair: sum over the shells of g e (f_C' - 2 eta d f_C), divided
// by r.  The result times (x_i - x_j) is the pair's pull on the centre (and minus that on the partner).
// `grow` is the centre's upstream row, `tj` the partner's type, `inv` = 1/r.
template <typename T>
__device__ __forceinline__ T bwd_radial_pair(const T* grow, int tj, T r, T inv)
{
    constexpr int kN = ShellWindow<T>::kShells;
    T g[kN], rs[kN];
    load_shell_window<T>(grow + tj * kNumRRs, ShellWindow<T>::first(r), g, rs);
    T fc, dfc;
    Fast<T>::cutoff_grad(r, static_cast<T>(kR_Rc_f), fc, dfc);
    return radial_shell_sum<T, kN>(g, rs, r, fc, dfc) * inv;           // dE/dr / r
}

// Both directions of a pair at once: centre c with partner j reads row c's block for j's type, centre j with
// partner c reads row j's block for c's type, and the two share r and with it every shell factor.  The result
// times (x_c - x_j) is the whole radial force on c from this pair, so that nothing has to be added to j: j
// receives the same when it is the centre.
template <typename T, bool kLibraryCutoff = false>
__device__ __forceinline__ T bwd_radial_pair_both(const T* grow_c, int tj, const T* grow_j, int tc, T r, T inv)
{
    constexpr int kN = ShellWindow<T>::kShells;
    T g[kN], w[kN], rs[kN];
    const int q0 = ShellWindow<T>::first(r);
    load_shell_window<T>(grow_c + tj * kNumRRs, q0, g, rs);
    load_shell_window<T>(grow_j + tc * kNumRRs, q0, w, rs);
    T fc, dfc;
    cutoff_grad_as<T, kLibraryCutoff>(r, static_cast<T>(kR_Rc_f), fc, dfc);
#pragma unroll
    for (int q = 0; q < kN; ++q) g[q] += w[q];
    return radial_shell_sum<T, kN>(g, rs, r, fc, dfc) * inv;
}

// The angular part of an upstream row is 320 elements = kRowPieces 16-byte pieces; a wavefront fetches it
// with kPieceRegs loads per lane (piece r * 64 + lane).
template <typename T, int kNB = kB> struct RowStage {
    static constexpr int kPerPiece = 16 / sizeof(T);                  // elements in a 16-byte piece
    static constexpr int kRowPieces = kAngular / kPerPiece;           // 80 (float) or 160 (double)
    static constexpr int kPieceRegs = (kRowPieces + 63) / 64;         // 2 or 3
    v4f st[kNB][kPieceRegs];

    // issues the loads for the rows of centres 0..nb-1; row_of(b) is wave-uniform
    template <typename RowOf>
    __device__ __forceinline__ void fetch(int lane, int nb, RowOf row_of)
    {
#pragma unroll
        for (int b = 0; b < kNB; ++b) {
            // Registers of centres beyond nb and of pieces beyond the row are never stored.  They are declared written
            // without an instruction: left unset they are "undefined" to the compiler, whose handling of that cost 30
            // registers here, and filling them with zeros costs 48 moves per batch.
#pragma unroll
            for (int r = 0; r < kPieceRegs; ++r) asm volatile("" : "=v"(st[b][r]));
            if (b < nb) {
                const global_v4f_ptr rowp = (global_v4f_ptr)(row_of(b) + kRadial);
#pragma unroll
                for (int r = 0; r < kPieceRegs; ++r)
                    if ((r + 1) * 64 <= kRowPieces || r * 64 + lane < kRowPieces) st[b][r] = rowp[r * 64 + lane];
            }
        }
    }
    // writes the fetched pieces into the pool, one 32-element block per type pair
    __device__ __forceinline__ void store(BwdPool<T, kNB>& pool, int lane, int nb) const
    {
#pragma unroll
        for (int b = 0; b < kNB; ++b) {
            if (b < nb) {
#pragma unroll
                for (int r = 0; r < kPieceRegs; ++r) {
                    const int piece = r * 64 + lane;
                    const int elem = piece * kPerPiece;
                    if ((r + 1) * 64 <= kRowPieces || piece < kRowPieces)
                        *reinterpret_cast<v4f*>(&pool.gst[b * kNumPairBlocks * kBlockStride + (elem >> 5) * kBlockStride + (elem & 31)]) = st[b][r];
                }
            }
        }
    }
};

// Copies of a batch's list that share the rounds: a pool of at most 32 (16) entries is walked by two (four)
// lanes per entry, lane = copy * span + entry, and copy h takes the rounds d = 1 + h, 1 + h + R, ...
__device__ __forceinline__ int round_copies(int total) { return total <= 16 ? 4 : total <= 32 ? 2 : 1; }

// Angular walk of a batch.  Lane = copy `copy` (of `copies`, a power of two; `span` = 64 / copies lanes each) of
// list entry `entry` of the pool, belonging to centre `bs` of the batch whose list starts at slot `pb` and has `m`
// entries (`live` = the lane has an entry).  In round d the entry pairs with entry (e + d) mod m of the same
// centre; after m/2 rounds every unordered pair has been visited once.  The force on the partner k goes to
// the copy's own pool.facc[copy * span + k] by plain read-add-write (the k of a centre are distinct within a round);
// the force on the lane's own entry is kept in registers.
// Returns the entry's total over all copies, in every copy's lane (zero for lanes without an entry).
// `type_of(sorted position)` gives an atom's type.
template <typename T, int kNB, typename TypeOf>
__device__ __forceinline__ typename Fast<T>::vec4 bwd_angular_rounds(BwdPool<T, kNB>& pool, int entry, int copy, int copies, bool live,
                                                     int bs, int pb, int m, TypeOf type_of)
{
    typedef typename Fast<T>::vec4 vec4;
    typedef typename Fast<T>::vec2 vec2;
    const int e = live ? entry - pb : 0;
    const int span = 64 / copies;
    const int mine = copy * span;          // this copy's slots of pool.facc
    // rounds: d = 1 .. (m-1)/2 for every entry; when m is even one more round for the lower half
    const int full = (m - 1) >> 1;
    const int rounds = live ? full + ((((m & 1) == 0) && (e < (m >> 1))) ? 1 : 0) : 0;
    const int max_rounds = kSkipAngular ? 0 : wave_max(rounds);
    const int self = live ? entry : 0;
    const vec4 vj = pool.nbr[self];
    const vec2 fj = pool.nbr_fc[self];
    const int tj = type_of(pool.nbr_idx[self]);
    const T inv_rj = Fast<T>::rcp(vj.w);
    const T* gbase = &pool.gst[bs * kNumPairBlocks * kBlockStride];
    T ajx = T(0), ajy = T(0), ajz = T(0);           // force on j, kept in registers

    for (int d0 = 1; d0 <= max_rounds; d0 += copies) {           // uniform trip count; copy h is at round d0 + h
        const int d = d0 + copy;
        const bool act = d <= rounds;
        int k = e + d;
        k -= (k >= m) ? m : 0;
        const int ks = act ? pb + k : 0;
        const vec4 vk = pool.nbr[ks];
        const vec2 fk = pool.nbr_fc[ks];
        const int tk = type_of(pool.nbr_idx[ks]);
        if (act) {
            const vec4* gp = reinterpret_cast<const vec4*>(gbase + pair_block(tj, tk) * kBlockStride);
            vec4 g[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) g[t] = gp[t];

            T c = vj.x * vk.x + vj.y * vk.y + vj.z * vk.z;
            c = fmin(fmax(c, T(-1)), T(1));
            const T cx = vj.y * vk.z - vj.z * vk.y;
            const T cy = vj.z * vk.x - vj.x * vk.z;
            const T cz = vj.x * vk.y - vj.y * vk.x;
            // cot(theta) = c/s has no limit for collinear triples (the angle has a cusp there, the
            // reference returns NaN): c s / (s^2 + eps) with eps = 1e-12 (float) or 1e-24 (double) equals
            // c/s to working precision a fraction of a degree off the line and goes to zero on it
            const T s2 = cx * cx + cy * cy + cz * cz;
            const T s = Fast<T>::sqrt_(s2);
            const T c_over_s = c * s * Fast<T>::rcp(s2 + Real<T>::kCotEps);
            const T rho = T(0.5) * (vj.w + vk.w);
            T Gs[4], dds[4];
#pragma unroll
            for (int sidx = 0; sidx < 4; ++sidx) {
                dds[sidx] = rho - static_cast<T>(kA_Rs_f[sidx]);
                Gs[sidx] = Fast<T>::gauss(static_cast<T>(kA_eta_f), dds[sidx]);
            }
            // X_s = sum_t g_ts A_t and Y_s = sum_t g_ts dA_t/dcos (without its factor 8)
            T Xs[4] = {T(0), T(0), T(0), T(0)}, Ys[4] = {T(0), T(0), T(0), T(0)};
            T bases[8];
            theta_bases<T>(c, s, bases);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const T ct = static_cast<T>(kCosTheta[t]), st = static_cast<T>(kSinTheta[t]);
                const T bs1 = bases[t];                              // 1 + cos(theta - theta_t)
                const T b2 = bs1 * bs1, b4 = b2 * b2;
                const T Am1 = b4 * b2 * bs1;                         // ^7
                const T At = Am1 * bs1;                              // ^8
                // (d/dcos) / 8 = Am1 (cos theta_t - cot sin theta_t); theta_0 = 0 exactly; in float theta_2 and theta_6
                // are pi/2 and 3 pi/2 to 8e-8, which leaves -cot and +cot (theta_4's sine stays: cot is unbounded)
                T dAt;
                if (t == 0) dAt = Am1;
                else if (sizeof(T) == 4 && t == 2) dAt = -c_over_s * Am1;
                else if (sizeof(T) == 4 && t == 6) dAt = c_over_s * Am1;
                else dAt = Am1 * fma(-c_over_s, st, ct);
                Xs[0] = fma(g[t].x, At, Xs[0]);
                Xs[1] = fma(g[t].y, At, Xs[1]);
                Xs[2] = fma(g[t].z, At, Xs[2]);
                Xs[3] = fma(g[t].w, At, Xs[3]);
                Ys[0] = fma(g[t].x, dAt, Ys[0]);
                Ys[1] = fma(g[t].y, dAt, Ys[1]);
                Ys[2] = fma(g[t].z, dAt, Ys[2]);
                Ys[3] = fma(g[t].w, dAt, Ys[3]);
            }
            // W0 = sum G_s X_s, Wc = 8 sum G_s Y_s, Wr = sum (dG_s/drho) X_s with dG/drho = -2 eta dd G
            const T gx0 = Gs[0] * Xs[0], gx1 = Gs[1] * Xs[1], gx2 = Gs[2] * Xs[2], gx3 = Gs[3] * Xs[3];
            const T W0 = (gx0 + gx1) + (gx2 + gx3);
            const T Wc = T(8) * fma(Gs[0], Ys[0], fma(Gs[1], Ys[1], fma(Gs[2], Ys[2], Gs[3] * Ys[3])));
            const T Wr = (T(-2) * static_cast<T>(kA_eta_f)) * fma(dds[0], gx0, fma(dds[1], gx1, fma(dds[2], gx2, dds[3] * gx3)));
            const T two_pow = T(0.0078125);
            const T P = two_pow * fj.x * fk.x;
            const T Fj = fma(P * T(0.5), Wr, two_pow * W0 * fj.y * fk.x);    // dE/dr_ij
            const T Fk = fma(P * T(0.5), Wr, two_pow * W0 * fj.x * fk.y);    // dE/dr_ik
            const T Fc = P * Wc;                                            // dE/dcos
            const T ij = Fc * inv_rj, ik = Fc * Fast<T>::rcp(vk.w);
            // force on j = -[Fj u_j + ij (u_k - c u_j)]; the bracket's second part is formed first, it
            // is small near the line where ij is large
            ajx = fma(-Fj, vj.x, fma(-ij, fma(-c, vj.x, vk.x), ajx));
            ajy = fma(-Fj, vj.y, fma(-ij, fma(-c, vj.y, vk.y), ajy));
            ajz = fma(-Fj, vj.z, fma(-ij, fma(-c, vj.z, vk.z), ajz));
            // force on k: in a round every lane of a centre holds a different k
            vec4 fk_acc = pool.facc[mine + ks];
            fk_acc.x = fma(-Fk, vk.x, fma(-ik, fma(-c, vk.x, vj.x), fk_acc.x));
            fk_acc.y = fma(-Fk, vk.y, fma(-ik, fma(-c, vk.y, vj.y), fk_acc.y));
            fk_acc.z = fma(-Fk, vk.z, fma(-ik, fma(-c, vk.z, vj.z), fk_acc.z));
            pool.facc[mine + ks] = fk_acc;
        }
        wave_lds_fence();
    }

    vec4 f = pool.facc[mine + self];
    f.x = live ? f.x + ajx : T(0);
    f.y = live ? f.y + ajy : T(0);
    f.z = live ? f.z + ajz : T(0);
    if (copies >= 2) {
        f.x += __shfl_xor(f.x, 32, 64);
        f.y += __shfl_xor(f.y, 32, 64);
        f.z += __shfl_xor(f.z, 32, 64);
    }
    if (copies == 4) {
        f.x += __shfl_xor(f.x, 16, 64);
        f.y += __shfl_xor(f.y, 16, 64);
        f.z += __shfl_xor(f.z, 16, 64);
    }
    return f;
}

}  // namespace khan
