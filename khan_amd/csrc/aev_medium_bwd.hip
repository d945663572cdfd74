// AEV backward (dL/dxyz) for molecules of up to 256 atoms that are too large for one wavefront (float32 from
// 33 atoms, float64 from 65): one workgroup of four wavefronts per molecule.
//
// The workgroup sorts the atoms by type into LDS once and zeroes the molecule's outputs.  Wavefronts
// then draw centres from a shared counter.  A wavefront collects centres into a batch while their
// angular partner lists fit the 64 entries of its pool (at most four), and for each centre it takes in:
//   scan + radial   the centre is tested against the sorted atoms 64 at a time; pairs inside the radial
//                   cutoff are queued, and whenever 64 are waiting a lane takes one pair and sums
//                   g e (f_C' - 2 eta d f_C) over the shells (float: the nine nearest to r) for both directions of the pair (the centre's
//                   row and the partner's row share every shell factor): that is the pair's whole pull on the
//                   centre, and nothing is added to the partner, which gets the same as a centre itself
//                   (per-pair atomic adds to the partners cost a quarter of the kernel);
// then for the batch:
//   stage           the 320 angular upstream values of each centre's row go to LDS by type pair;
//   angular         the round-robin walk shared with the small-molecule kernel: lane = list entry,
//                   partner forces by conflict-free read-add-write in LDS;
//   gather          every list entry adds its total to its atom, every centre gets minus its list's sum.
// Forces go to the output arrays with global atomics (a molecule's atoms are shared by four wavefronts).
// A centre with more than 64 angular partners is handled by the general per-centre routine.
// Reference: gpu_featurizer/kernel_cpu.cpp:217-366.
#include <type_traits>

#include "aev_bwd_batch.h"
#include "aev_large.h"

namespace khan {

namespace {

constexpr int kChunks = kMediumMaxAtoms / 64;
constexpr int kTypeShift = 28;     // large molecules: a radial queue entry is a sorted position with the atom's type above it
// centres per batch: four, so that the pools of the four wavefronts leave room for four workgroups on a CU in float
// (LDS 39.6 KB; 128 registers) and two in double (76 KB; 256 registers) -- the shorter batches fill fewer lanes, the
// additional wavefronts per SIMD hide more (dense boxes: float 4 % faster than six-centre batches at three workgroups,
// double 23 % faster than at one).
template <typename T> constexpr int kMedBwdCentres = 4;

// Where a molecule's forces are summed.
// kLocal = false: hardware atomics on the output arrays (zeroed by the workgroup first).  The fastest form, and the
// only one for molecules of more than 256 atoms, which several workgroups share; the order of the additions, and with
// it the last bits of the gradients, varies from run to run, and the output arrays must be in memory that supports
// the atomics (ordinary device allocations).
// kLocal = true (up to 256 atoms, on request: khan_set_reproducible_gradients): in LDS, one array per wavefront, by
// plain read-add-write -- every instruction that adds is arranged so that its lanes hit distinct atoms -- the four
// arrays added up in a fixed order at the end and every gradient stored once: no atomics, no pre-zeroed output, and,
// with the centres dealt to the wavefronts by their position, the same result bit for bit on every run.  Each radial
// pair is then evaluated once and pulls on both its atoms (with atomics it is evaluated from both ends, because
// per-pair atomic adds to the partners cost more than the arithmetic they save).  The arrays take 12 KB (float), which
// leaves three workgroups per CU instead of four: measured 9 % slower on dense boxes (0.90 -> 0.98 ms), with
// the kernel's HBM traffic down from 2.14 to 1.07 times its algorithmic bytes.
template <typename T, bool kOn> struct ForceLds {};
template <typename T> struct ForceLds<T, true> {
    T f[4][3][kMediumMaxAtoms];            // [wavefront][component][sorted position]
    unsigned short where[kMediumMaxAtoms]; // index inside the molecule -> sorted position
};

template <typename T, bool kLarge = false, bool kLocal = false>
struct __align__(16) MedBwdShared {
    ForceLds<T, kLocal> force;
    typename Fast<T>::vec4 atom[kMediumMaxAtoms];   // x, y, z, type (sorted order)
    unsigned row_lo[kMediumMaxAtoms];      // address of the atom's upstream row
    unsigned row_hi[kMediumMaxAtoms];
    unsigned short orig[kMediumMaxAtoms];  // sorted position -> index inside the molecule
    int wcount[4][4];                      // atoms of each type held by each wavefront before the sort
    int next;                              // next centre (sorted position) to hand out
};
// above 256 atoms the sorted atoms are in device memory (aev_large.h); the list entries' sorted positions no
// longer fit a byte and are kept here, one array per wavefront (the pool's byte array then holds the types)
template <typename T>
struct __align__(16) MedBwdShared<T, true, false> {
    int pos[4][64];
    int next;                              // centres handed out so far by this workgroup
};

// With kLarge the kernel takes the molecules of more than 256 atoms: the atoms come type-sorted from `sorted`, the
// workgroups of one grid column (blockIdx.y = 0 .. gridDim.y - 1) share a molecule's centres, and the gradients were
// zeroed by the kernel that sorted the atoms.
template <typename T, bool kLarge = false, bool kLocal = false>
__global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? (kLocal ? 3 : 4) : (kLocal ? 1 : 2), sizeof(T) == 4 ? (kLocal ? 3 : 4) : (kLocal ? 1 : 2))))
void aev_bwd_medium_kernel(
    const T* __restrict__ X, const T* __restrict__ Y, const T* __restrict__ Z,
    const int32_t* __restrict__ A, const int32_t* __restrict__ MOs,
    const int32_t* __restrict__ MACs, int32_t n_mols, const int32_t* __restrict__ SIs,
    Buckets<const T> gin, T* __restrict__ gX, T* __restrict__ gY, T* __restrict__ gZ, int min_atoms,
    const int32_t* __restrict__ order, bool walk_in_order, const SortedAtoms<T> sorted)
{
    typedef typename Fast<T>::vec4 vec4;
    typedef typename std::conditional<kLarge, int, unsigned short>::type idx_t;     // a sorted position in the radial queue
    static_assert(!(kLarge && kLocal), "forces in LDS: molecules of up to 256 atoms only");
    __shared__ MedBwdShared<T, kLarge, kLocal> M;
    constexpr int kMB = kMedBwdCentres<T>;
    // the double kernel for 65-256 atoms runs at 256 registers (two workgroups per compute unit): with the cutoff's
    // polynomial constants resident it spills 21 of them and is 8 % slower than with the library's cos and sin
    constexpr bool kLibraryCutoff = sizeof(T) == 8 && !kLarge && !kLocal;
    __shared__ BwdPool<T, kMB> pools[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    BwdPool<T, kMB>& P = pools[wave];
    const LaneConsts<T> L = lane_consts<T>(lane);
    const unsigned long long lt_mask = (1ull << lane) - 1ull;

    __shared__ unsigned long long want[4];
    for_each_molecule_in_range(MACs, n_mols, min_atoms, kLarge ? INT32_MAX : kMediumMaxAtoms, want, walk_in_order ? order : nullptr,
                               order ? order + n_mols : nullptr, [&](int mol) {
        const int n = uniform(MACs[mol]);
        const int off = uniform(MOs[mol]);
        int tb1, tb2, tb3;                     // sorted position of the first C, N, O atom

        // ------------------------------------------------------------ load, sort by type into LDS, zero outputs
        if constexpr (kLarge) {
            tb1 = tb2 = tb3 = 0;               // (the sorted atoms are not in order of type: types come with the atoms)
            if (tid == 0) M.next = 0;
            __syncthreads();
        } else {
        const bool have = tid < n;
        T x = T(0), y = T(0), z = T(0);
        int type = 0;
        unsigned long long rowbits = 0;
        if (have) {
            x = X[off + tid];
            y = Y[off + tid];
            z = Z[off + tid];
            type = fold_type(A[off + tid]);
            rowbits = reinterpret_cast<unsigned long long>(gin.p[type] + static_cast<size_t>(SIs[off + tid]) * kFeats);
            if constexpr (!kLocal) {
                gX[off + tid] = T(0);
                gY[off + tid] = T(0);
                gZ[off + tid] = T(0);
            }
        }
        if constexpr (kLocal) {
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int k = 0; k < 3; ++k) M.force.f[w][k][tid] = T(0);
        }
        unsigned long long tmask[4];
#pragma unroll
        for (int a = 0; a < 4; ++a) tmask[a] = wave_ballot(have && type == a);
        if (lane < 4) M.wcount[wave][lane] = popc64(lane == 0 ? tmask[0] : lane == 1 ? tmask[1] : lane == 2 ? tmask[2] : tmask[3]);
        if (tid == 0) M.next = 0;
        __syncthreads();
        int tbase[4];
        {
            int run = 0;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                tbase[a] = run;
                run += M.wcount[0][a] + M.wcount[1][a] + M.wcount[2][a] + M.wcount[3][a];
            }
        }
        if (have) {
            int before = 0;                     // atoms of my type held by earlier wavefronts
            for (int w = 0; w < wave; ++w) before += M.wcount[w][type];
            const unsigned long long mine = type == 0 ? tmask[0] : type == 1 ? tmask[1] : type == 2 ? tmask[2] : tmask[3];
            const int dest = sel4(type, tbase[0], tbase[1], tbase[2], tbase[3]) + before + popc64(mine & lt_mask);
            M.atom[dest] = Fast<T>::make4(x, y, z, static_cast<T>(type));
            M.row_lo[dest] = static_cast<unsigned>(rowbits & 0xffffffffull);
            M.row_hi[dest] = static_cast<unsigned>(rowbits >> 32);
            M.orig[dest] = static_cast<unsigned short>(tid);
            if constexpr (kLocal) M.force.where[tid] = static_cast<unsigned short>(dest);
        }
        __syncthreads();       // sorted arrays complete; the zeroed outputs are visible before any atomic add
        tb1 = tbase[1];
        tb2 = tbase[2];
        tb3 = tbase[3];
        }
        auto type_of = [&](int sorted_idx) { return (sorted_idx >= tb1) + (sorted_idx >= tb2) + (sorted_idx >= tb3); };
        auto atom_at = [&](int sorted_idx) -> vec4 {
            if constexpr (kLarge) return sorted.atom[off + sorted_idx];
            else return M.atom[sorted_idx];
        };
        auto row_bits_of = [&](int sorted_idx, int type) -> unsigned long long {     // per-lane index, and that atom's type
            if constexpr (kLarge) {
                const T* const bucket = type == 0 ? gin.p[0] : type == 1 ? gin.p[1] : type == 2 ? gin.p[2] : gin.p[3];
                return reinterpret_cast<unsigned long long>(bucket + static_cast<size_t>(sorted.aux[off + sorted_idx].y) * kFeats);
            } else {
                return (static_cast<unsigned long long>(M.row_hi[sorted_idx]) << 32) | M.row_lo[sorted_idx];
            }
        };
        auto row_of = [&](int sorted_idx) -> const T* {            // wave-uniform index
            int type = 0;
            if constexpr (kLarge) type = static_cast<int>(sorted.atom[off + sorted_idx].w);
            const unsigned long long bits = row_bits_of(sorted_idx, type);
            const unsigned lo = static_cast<unsigned>(uniform(static_cast<int>(bits & 0xffffffffull)));
            const unsigned hi = static_cast<unsigned>(uniform(static_cast<int>(bits >> 32)));
            return reinterpret_cast<const T*>((static_cast<unsigned long long>(hi) << 32) | lo);
        };
        auto orig_of = [&](int sorted_idx) -> int {                // per-lane index
            if constexpr (kLarge) return sorted.aux[off + sorted_idx].x;
            else return M.orig[sorted_idx];
        };
        // per-lane target; with forces in LDS the caller sees to it that the lanes of one call hit distinct atoms
        auto add_force = [&](int sorted_idx, T fx, T fy, T fz) {
            if constexpr (kLocal) {
                M.force.f[wave][0][sorted_idx] += fx;
                M.force.f[wave][1][sorted_idx] += fy;
                M.force.f[wave][2][sorted_idx] += fz;
            } else {
                const int g = off + orig_of(sorted_idx);
                atomicAdd(&gX[g], fx);
                atomicAdd(&gY[g], fy);
                atomicAdd(&gZ[g], fz);
            }
        };

        // Radial pairs are queued and worked off 64 at a time: only about an eighth of the (centre, partner)
        // pairs of a large molecule lie inside the radial cutoff, so evaluating them where they are found
        // would leave most lanes idle.  The queue lives in the pool's staging area, which is free while a
        // batch is being collected; it is emptied before the batch's upstream rows are staged.
        vec4* const q_d = reinterpret_cast<vec4*>(P.gst);                          // 128 x (dx, dy, dz, r)
        idx_t* const q_j = reinterpret_cast<idx_t*>(q_d + 128);                    // partner (sorted position)
        idx_t* const q_c = q_j + 128;                                              // centre (sorted position)
        int qn = 0;
        auto radial_work_off = [&](int count) {      // entries 0..count-1, count <= 64
            T fx = T(0), fy = T(0), fz = T(0);
            int c = -1, j = 0;
            if (lane < count) {
                const vec4 e = q_d[lane];
                j = q_j[lane];
                c = q_c[lane];
                int tj, tc;
                if constexpr (kLarge) {            // the queue carries the types in the four high bits
                    tj = j >> kTypeShift;
                    tc = c >> kTypeShift;
                    j &= (1 << kTypeShift) - 1;
                    c &= (1 << kTypeShift) - 1;
                } else {
                    tj = type_of(j);
                    tc = type_of(c);
                }
                const T* grow_c = reinterpret_cast<const T*>(row_bits_of(c, tc));
                const T* grow_j = reinterpret_cast<const T*>(row_bits_of(j, tj));
                const T inv = Fast<T>::rcp(e.w);
                // the pair's pull on the centre from both rows.  With forces in LDS the pair is queued once (by its
                // centre of lower sorted position) and the partner gets minus this below; otherwise the partner gets
                // its share when it is the centre
                const T sc = bwd_radial_pair_both<T, kLibraryCutoff>(grow_c, tj, grow_j, tc, e.w, inv);
                fx = sc * e.x;
                fy = sc * e.y;
                fz = sc * e.z;
            }
            // The pairs of one centre are a run of lanes (the queue is filled centre after centre): one add-scan
            // per component, and the last lane of every run adds the difference of two prefix values to its
            // centre -- one add per centre and component, issued for all centres of the step at once.
            const T px = group_sum_to_last_lane(fx, 6), py = group_sum_to_last_lane(fy, 6), pz = group_sum_to_last_lane(fz, 6);
            const int c_prev = __builtin_amdgcn_ds_bpermute(max(lane - 1, 0) << 2, c);
            const int c_next = __builtin_amdgcn_ds_bpermute(min(lane + 1, 63) << 2, c);
            const bool in_q = lane < count;
            const unsigned long long starts = wave_ballot(in_q && (lane == 0 || c_prev != c));
            const bool run_end = in_q && (lane == count - 1 || c_next != c);
            // first lane of this lane's run: the highest start at or below the lane
            const unsigned long long below = starts & ((lane == 63) ? ~0ull : ((2ull << lane) - 1ull));
            const int first = below ? 63 - __clzll(static_cast<long long>(below)) : 0;
            const int at = max(first - 1, 0) << 2;
            const T qx = lane_fetch(px, at), qy = lane_fetch(py, at), qz = lane_fetch(pz, at);
            if (run_end) {
                const bool whole = first == 0;
                add_force(c, whole ? px : px - qx, whole ? py : py - qy, whole ? pz : pz - qz);
            }
            if constexpr (kLocal) {
                // the partners: run after run, because the partners of one centre are distinct atoms and those of two
                // centres need not be
                wave_lds_fence();
                for (unsigned long long rs = starts; rs;) {
                    const int b0 = lowest_bit(rs);
                    rs &= rs - 1;
                    const int b1 = rs ? lowest_bit(rs) : count;
                    if (lane >= b0 && lane < b1) add_force(j, -fx, -fy, -fz);
                    wave_lds_fence();
                }
            }
        };
        auto radial_drain = [&]() {
            wave_lds_fence();
            while (qn > 0) {
                const int take = min(qn, 64);
                radial_work_off(take);
                const int rest = qn - take;
                vec4 e = Fast<T>::make4(T(0), T(0), T(0), T(1));
                idx_t ej = 0, ec = 0;
                if (lane < rest) {
                    e = q_d[64 + lane];
                    ej = q_j[64 + lane];
                    ec = q_c[64 + lane];
                }
                wave_lds_fence();
                if (lane < rest) {
                    q_d[lane] = e;
                    q_j[lane] = ej;
                    q_c[lane] = ec;
                }
                wave_lds_fence();
                qn = rest;
            }
        };
        // a full wave of queued pairs: work it off, keep the rest
        auto radial_work_off_full = [&]() {
            wave_lds_fence();
            radial_work_off(64);
            const int rest = qn - 64;
            vec4 e = Fast<T>::make4(T(0), T(0), T(0), T(1));
            idx_t ej = 0, ec = 0;
            if (lane < rest) {
                e = q_d[64 + lane];
                ej = q_j[64 + lane];
                ec = q_c[64 + lane];
            }
            wave_lds_fence();
            if (lane < rest) {
                q_d[lane] = e;
                q_j[lane] = ej;
                q_c[lane] = ec;
            }
            wave_lds_fence();
            qn = rest;
        };

        int dealt = 0;             // (forces in LDS) centres this wavefront has taken: it takes every fourth, by position
        int pending = -1;          // a centre that was drawn but did not fit the previous batch
        int scanned = -1;          // (large molecules) the centre whose radial pairs were queued last
        for (;;) {
            // ------------------------------------------------ collect a batch of centres
            int nb = 0, used = 0;
            int pfv = 0, cv = 0;   // lane k: first pool slot and sorted position of centre k of the batch
            P.facc[lane] = Fast<T>::make4(T(0), T(0), T(0), T(0));
            while (nb < kMB) {
                int c = pending;
                pending = -1;
                if (c < 0) {
                    if constexpr (kLocal) {
                        c = wave + 4 * dealt++;
                    } else {
                        int drawn = 0;
                        if (lane == 0) drawn = atomicAdd(&M.next, 1);
                        c = uniform(drawn);
                        if constexpr (kLarge) c = static_cast<int>(blockIdx.y) + static_cast<int>(gridDim.y) * c;
                    }
                }
                if (c >= n) break;
                const vec4 ai = atom_at(c);
                int m_c = 0;
                bool too_many;
                if constexpr (kLarge) {
                    // One pass over the partners, 64 at a time: list entries are written behind the batch's as they
                    // are found (a centre that turns out not to fit leaves them there, unused, and opens the next
                    // batch, where it is scanned again; its radial pairs are queued the first time only).
                    const bool again = c == scanned;
                    int pos = used;
                    auto scan_chunk = [&](int jc, const vec4 aj) {
                        const int j = jc + lane;
                        const T ddx = ai.x - aj.x, ddy = ai.y - aj.y, ddz = ai.z - aj.z;
                        const T rr = Fast<T>::sqrt_rn(ddx * ddx + ddy * ddy + ddz * ddz);
                        const bool valid = (j < n) && (j != c);
                        const unsigned long long mRb = wave_ballot(!kSkipRadial && !again && valid && (rr < kR_Rc_f) && (rr > T(0)));
                        const unsigned long long mAb = wave_ballot(valid && (rr < kA_Rc_f) && (rr > T(0)));
                        if ((mAb >> lane) & 1ull) {
                            const int p = pos + popc64(mAb & lt_mask);
                            if (p < 64) {
                                P.nbr[p] = Fast<T>::make4(ddx, ddy, ddz, rr);
                                P.nbr_idx[p] = static_cast<unsigned char>(static_cast<int>(aj.w));      // the partner's type
                                M.pos[wave][p] = j;
                            }
                        }
                        pos += popc64(mAb);
                        m_c += popc64(mAb);
                        if ((mRb >> lane) & 1ull) {
                            const int p = qn + popc64(mRb & lt_mask);
                            q_d[p] = Fast<T>::make4(ddx, ddy, ddz, rr);
                            q_j[p] = static_cast<idx_t>(j | (static_cast<int>(aj.w) << kTypeShift));
                            q_c[p] = static_cast<idx_t>(c | (static_cast<int>(ai.w) << kTypeShift));
                        }
                        qn += popc64(mRb);
                        if (qn >= 64) radial_work_off_full();
                    };
                    // 64 chunks' boxes are tested against the centre at a time (one per lane); the chunks that reach into
                    // the radial cutoff are scanned, four chunks' loads in flight at a time
                    const float cx = static_cast<float>(ai.x), cy = static_cast<float>(ai.y), cz = static_cast<float>(ai.z);
                    const int n_chunks = (n + 63) >> 6;
                    const float4* const boxes = sorted.box + 2 * chunk_base(off, mol);
                    for (int ch0 = 0; ch0 < n_chunks; ch0 += 64) {
                        unsigned long long near = wave_ballot(chunk_in_reach(boxes, ch0 + lane, n_chunks, cx, cy, cz));
                        while (near) {
                            int ch[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                ch[u] = -1;
                                if (near) {
                                    ch[u] = ch0 + lowest_bit(near);
                                    near &= near - 1;
                                }
                            }
                            vec4 at[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) at[u] = atom_at(min(max(ch[u], 0) * 64 + lane, n - 1));
#pragma unroll
                            for (int u = 0; u < 4; ++u)
                                if (ch[u] >= 0) scan_chunk(ch[u] * 64, at[u]);
                        }
                    }
                    scanned = c;
                    too_many = m_c > 64;
                    if (!too_many && nb > 0 && used + m_c > 64) {       // full: this centre opens the next batch
                        pending = c;
                        break;
                    }
                } else {
                // first pass over the partners: who is inside the cutoffs
                T dx[kChunks], dy[kChunks], dz[kChunks], r[kChunks];
                unsigned long long mA[kChunks], mR[kChunks];
#pragma unroll
                for (int ch = 0; ch < kChunks; ++ch) {
                    mA[ch] = 0ull;
                    mR[ch] = 0ull;
                    dx[ch] = dy[ch] = dz[ch] = T(0);
                    r[ch] = T(1);
                    if (ch * 64 < n) {
                        const int j = ch * 64 + lane;
                        const vec4 aj = M.atom[j];
                        dx[ch] = ai.x - aj.x;
                        dy[ch] = ai.y - aj.y;
                        dz[ch] = ai.z - aj.z;
                        r[ch] = Fast<T>::sqrt_rn(dx[ch] * dx[ch] + dy[ch] * dy[ch] + dz[ch] * dz[ch]);
                        const bool valid = (j < n) && (j != c);
                        // r = 0: a coincident atom exerts no force; with forces in LDS a pair is queued by its lower centre only
                        mR[ch] = wave_ballot(!kSkipRadial && valid && (r[ch] < kR_Rc_f) && (r[ch] > T(0)) && (!kLocal || j > c));
                        mA[ch] = wave_ballot(valid && (r[ch] < kA_Rc_f) && (r[ch] > T(0)));
                        m_c += popc64(mA[ch]);
                    }
                }
                too_many = m_c > 64;                   // more partners than a pool holds
                if (!too_many && nb > 0 && used + m_c > 64) {       // full: this centre opens the next batch
                    pending = c;
                    break;
                }
                // second pass: list entries; radial pairs join the queue
                int pos = used;
#pragma unroll
                for (int ch = 0; ch < kChunks; ++ch) {
                    if (ch * 64 < n) {
                        const int j = ch * 64 + lane;
                        if (!too_many && ((mA[ch] >> lane) & 1ull)) {
                            // the entry as found; unit vector and cutoff are worked out once per centre below, on
                            // the compacted list, not once per chunk on every lane
                            const int p = pos + popc64(mA[ch] & lt_mask);
                            P.nbr[p] = Fast<T>::make4(dx[ch], dy[ch], dz[ch], r[ch]);
                            P.nbr_idx[p] = static_cast<unsigned char>(j);
                        }
                        pos += popc64(mA[ch]);
                        if ((mR[ch] >> lane) & 1ull) {
                            const int p = qn + popc64(mR[ch] & lt_mask);
                            q_d[p] = Fast<T>::make4(dx[ch], dy[ch], dz[ch], r[ch]);
                            q_j[p] = static_cast<unsigned short>(j);
                            q_c[p] = static_cast<unsigned short>(c);
                        }
                        qn += popc64(mR[ch]);
                        if (qn >= 64) radial_work_off_full();
                    }
                }
                }
                if (!too_many) {
                    wave_lds_fence();
                    if (lane < m_c) {
                        const vec4 d = P.nbr[used + lane];
                        const T inv = Fast<T>::rcp(d.w);
                        T fc, dfc;
                        cutoff_grad_as<T, kLibraryCutoff>(d.w, static_cast<T>(kA_Rc_f), fc, dfc);
                        P.nbr[used + lane] = Fast<T>::make4(d.x * inv, d.y * inv, d.z * inv, d.w);
                        P.nbr_fc[used + lane] = Fast<T>::make2(fc, dfc);
                    }
                }
                if (too_many) {
                    // the general per-centre routine does this centre's angular part alone (its radial pairs are
                    // in the queue like everyone's)
                    const int i_orig = uniform(orig_of(c));
                    radial_drain();                    // the routine uses the staging area as scratch
                    bwd_center_generic<T>(L, lane, X, Y, Z, A, off, n, i_orig, P.gst, row_of(c),
                                              [&](int atom, T fx, T fy, T fz) {
                                                  if constexpr (kLocal) {
                                                      // (lanes may meet on an atom here: LDS atomics, whose order within
                                                      // an instruction is the hardware's)
                                                      const int sp = M.force.where[atom];
                                                      atomicAdd(&M.force.f[wave][0][sp], fx);
                                                      atomicAdd(&M.force.f[wave][1][sp], fy);
                                                      atomicAdd(&M.force.f[wave][2][sp], fz);
                                                  } else {
                                                      atomicAdd(&gX[off + atom], fx);
                                                      atomicAdd(&gY[off + atom], fy);
                                                      atomicAdd(&gZ[off + atom], fz);
                                                  }
                                              },
                                              false);
                    wave_lds_fence();
                    continue;
                }
                if (lane == nb) {
                    pfv = used;
                    cv = c;
                }
                used += m_c;
                ++nb;
            }
            radial_drain();                          // frees the staging area
            if (nb == 0) break;
            if (lane >= nb) pfv = used;              // lanes nb.. hold the end of the pool

            // ---- the angular upstream blocks of the batch's rows go to LDS (80 x 16 bytes per row)
            {
                RowStage<T, kMB> stage;
                stage.fetch(lane, nb, [&](int b) { return row_of(lane_read(cv, b)); });
                stage.store(P, lane, nb);
            }
            wave_lds_fence();

            // ------------------------------------------------ angular: lane = list entry (centre, partner j)
            const int pf1 = lane_read(pfv, 1), pf2 = lane_read(pfv, 2), pf3 = lane_read(pfv, 3),
                      pf4 = lane_read(pfv, 4), pf5 = lane_read(pfv, 5), pf6 = lane_read(pfv, 6);
            const int total = used;
            // a short pool is walked by two or four lanes per entry, which share its rounds
            const int copies = round_copies(total), span = 64 / copies;
            const int entry = lane & (span - 1), copy = lane / span;
            const int b = (entry >= pf1) + (entry >= pf2) + (entry >= pf3) + (entry >= pf4) + (entry >= pf5);
            const int bs = entry < total ? b : 0;
            const int pb = sel6(bs, 0, pf1, pf2, pf3, pf4, pf5);
            const int m = sel6(bs, pf1, pf2, pf3, pf4, pf5, pf6) - pb;
            // (the byte per list entry: the partner's sorted position, or for large molecules its type)
            const vec4 f = bwd_angular_rounds<T>(P, entry, copy, copies, entry < total, bs, pb, m,
                                                 [&](int v) { if constexpr (kLarge) return v; else return type_of(v); });
            const bool live = lane < total;       // from here on one lane per entry again

            // ------------------------------------------------ gather
            if constexpr (kLocal) {
                // centre after centre: the partners of one centre are distinct atoms
                const int target = P.nbr_idx[live ? lane : 0];
                for (int bb = 0; bb < nb; ++bb) {
                    if (live && bs == bb) add_force(target, f.x, f.y, f.z);
                    wave_lds_fence();
                }
            } else if (live) {
                if constexpr (kLarge) add_force(M.pos[wave][lane], f.x, f.y, f.z);
                else add_force(P.nbr_idx[lane], f.x, f.y, f.z);
            }
            {
                // a centre's list is a run of lanes: its sum is the difference of two values of an add-scan,
                // and lane b adds centre b's
                const T px = group_sum_to_last_lane(live ? f.x : T(0), 6);
                const T py = group_sum_to_last_lane(live ? f.y : T(0), 6);
                const T pz = group_sum_to_last_lane(live ? f.z : T(0), 6);
                const int lo = __builtin_amdgcn_ds_bpermute(min(lane, 63) << 2, pfv);          // pfv of lane b = first slot of centre b
                const int hi = __builtin_amdgcn_ds_bpermute(min(lane + 1, 63) << 2, pfv);
                const int at_hi = max(hi - 1, 0) << 2, at_lo = max(lo - 1, 0) << 2;
                T sx = lane_fetch(px, at_hi), sy = lane_fetch(py, at_hi), sz = lane_fetch(pz, at_hi);
                const T qx = lane_fetch(px, at_lo), qy = lane_fetch(py, at_lo), qz = lane_fetch(pz, at_lo);
                if (lo > 0) {
                    sx -= qx;
                    sy -= qy;
                    sz -= qz;
                }
                if (lane < nb && hi > lo) add_force(cv, -sx, -sy, -sz);      // cv of lane b = centre b
            }
            wave_lds_fence();
        }
        if constexpr (kLocal) {
            __syncthreads();  // every wavefront's forces are complete
            if (tid < n) {
                const int g = off + M.orig[tid];
                gX[g] = (M.force.f[0][0][tid] + M.force.f[1][0][tid]) + (M.force.f[2][0][tid] + M.force.f[3][0][tid]);
                gY[g] = (M.force.f[0][1][tid] + M.force.f[1][1][tid]) + (M.force.f[2][1][tid] + M.force.f[3][1][tid]);
                gZ[g] = (M.force.f[0][2][tid] + M.force.f[1][2][tid]) + (M.force.f[2][2][tid] + M.force.f[3][2][tid]);
            }
        }
        __syncthreads();      // the next molecule reuses the sorted arrays
    });
}

}  // namespace

template <typename T>
hipError_t launch_bwd_medium(const T* X, const T* Y, const T* Z, const int32_t* A,
                             const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                             const int32_t* SIs, Buckets<const T> g, T* gX, T* gY,
                             T* gZ, int min_atoms, const int32_t* order, bool walk_in_order, bool reproducible,
                             hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    // workgroups walk the molecules with the grid's stride and skip those of other sizes
    // (in float64 the working set lets one workgroup run per CU: a smaller grid costs less when it only skips)
    const int32_t cap = sizeof(T) == 4 ? 4096 : 1024;
    const unsigned blocks = static_cast<unsigned>(n_mols < cap ? n_mols : cap);
    if (reproducible)
        aev_bwd_medium_kernel<T, false, true><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ, min_atoms,
                                                                                   order, walk_in_order, SortedAtoms<T>{});
    else
        aev_bwd_medium_kernel<T><<<dim3(blocks), dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ, min_atoms,
                                                                      order, walk_in_order, SortedAtoms<T>{});
    return hipGetLastError();
}

// Molecules of more than 256 atoms: the sort into `scratch` (large_scratch_bytes), which also zeroes their gradients,
// then the kernel above with the centres of a molecule spread over the workgroups of a grid column.
template <typename T>
hipError_t launch_bwd_large(const T* X, const T* Y, const T* Z, const int32_t* A,
                            const int32_t* MOs, const int32_t* MACs, int32_t n_mols,
                            const int32_t* SIs, Buckets<const T> g, T* gX, T* gY, T* gZ,
                            const int32_t* order, void* scratch, int64_t n_atoms, hipStream_t stream)
{
    if (n_mols <= 0) return hipSuccess;
    const SortedAtoms<T> sorted = carve_sorted_atoms<T>(scratch, n_atoms, n_mols, false);
    const hipError_t e = launch_large_sort<T>(X, Y, Z, A, MOs, MACs, n_mols, SIs, nullptr, nullptr, nullptr, gX, gY, gZ, order,
                                              sorted, stream);
    if (e != hipSuccess) return e;
    const dim3 grid = large_grid(n_mols);
    aev_bwd_medium_kernel<T, true><<<grid, dim3(256), 0, stream>>>(X, Y, Z, A, MOs, MACs, n_mols, SIs, g, gX, gY, gZ,
                                                                  kMediumMaxAtoms + 1, order, false, sorted);
    return hipGetLastError();
}

template hipError_t launch_bwd_medium<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const float>, float*, float*, float*, int, const int32_t*, bool, bool, hipStream_t);
template hipError_t launch_bwd_medium<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const double>, double*, double*, double*, int, const int32_t*, bool, bool, hipStream_t);

template hipError_t launch_bwd_large<float>(const float*, const float*, const float*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const float>, float*, float*, float*, const int32_t*, void*, int64_t, hipStream_t);
template hipError_t launch_bwd_large<double>(const double*, const double*, const double*, const int32_t*, const int32_t*, const int32_t*, int32_t, const int32_t*, Buckets<const double>, double*, double*, double*, const int32_t*, void*, int64_t, hipStream_t);

}  // namespace khan
