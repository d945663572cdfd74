// The whole atomic network of the reference's default size, 384-128-128-64-1 with CELU (khan/model/nn.py:38-68,
// khan/model/activations.py:63-65; sizes: khan/inference/energy_server.py:121), for the four atom types in ONE launch,
// forward and -- on request -- back to the feature rows:
//     a1 = celu(x W1 + b1), a2 = celu(a1 W2 + b2), a3 = celu(a2 W3 + b3), e = a3 w4 + b4          (per feature row x)
//     g3 = s w4^T .* celu'(a3), g2 = (g3 W3^T) .* celu'(a2), g1 = (g2 W2^T) .* celu'(a1), dx = g1 W1^T
// with s the gradient with respect to each row's value e (1 when none is given: the gradient of the sum of the values,
// which is what forces need).  A feature row is read once and its gradient written once: the activations of a tile of
// rows never leave the compute unit.  Layer by layer the same pass moves 2.9 GB forward and 3.7 GB back per 767,292
// rows (every activation written, read again by the next layer and once more on the way back); this one moves the rows
// and their gradients, 2.4 GB, and the values.
//
// One workgroup of four wavefronts owns 64 rows; two workgroups share a compute unit and, having no barriers in common,
// fill each other's waits.  The products run on the 16-bit matrix instructions
// (v_mfma_f32_32x32x16_f16, sixteen times the rate of the float32 ones) with every float32 operand split into two
// half-precision parts:
//     x = h + 2^-11 l,   h = half(x),   l = half(2^11 (x - h))
// h carries 11 significant bits, x - h is exact in float32 and at most 2^-12 |x|, and l carries its 11 leading bits:
// |x - h - 2^-11 l| <= 2^-24 |x|, the rounding of float32 itself.  The residual is scaled by 2^11 so that it has
// x's exponent and not one twelve binary orders below it, where half precision would run out of exponent for every
// |x| < 0.25.  Of the four partial products of x w three are kept, each an exact 22-bit product accumulated in
// float32, in two accumulators:
//     hi += h_x h_w,   lo += h_x l_w + l_x h_w,   x w ~ hi + 2^-11 lo      (left out: l_x l_w 2^-22 <= 2^-24 |x w|)
// which is a float32 product to float32 accuracy (three terms of 2^-24 |x w| each) from three matrix instructions;
// the three-way bfloat16 split of dense_first.hip needs six.  What it costs is range: half precision ends at 65,504,
// so an operand (feature, activation, weight) of that size or more gives NaN -- never a wrong finite number -- and an
// |x| below 6e-5 keeps an absolute accuracy of 2^-36 instead of a relative one.  On the way back the gradient is
// carried for a unit upstream factor and multiplied by the row's factor only when it is stored (the pass is linear
// in it), so that the gradients' size inside the kernel does not depend on the caller's loss scale.
// A wavefront holds all 64 rows of 32 columns of a layer's 64 x 128 output
// (32 x 32 of the 64 x 64 one) in accumulator registers, and keeps its part of a1, a2 and a3 in registers for the way
// back, where the gradients arrive in the same places.  Between layers the activations (gradients) go to LDS already
// split, as two planes [row][k] of half precision: the next product's row operand, read straight from there.  The weights
// do not pass through LDS: every wavefront loads its operands of a chunk of 16 k straight into registers (layer_product)
// -- from the chunks the caller has had split once beforehand (launch_networks_pack), or from the float32 weights, which
// a lane then splits itself.  Layer 1's feature rows, float32 in memory, go through a double-buffered LDS stage in the
// space the activation planes take later.  LDS: 35 KB per workgroup; 2 wavefronts per SIMD (the accumulators and the
// saved activations take 200 registers).
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

namespace {

typedef float v4 __attribute__((ext_vector_type(4)));
typedef float v16 __attribute__((ext_vector_type(16)));
typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef float f2v __attribute__((ext_vector_type(2)));

constexpr int kDepthRows = 4;       // chunks of weights in flight in layer 1 (= two pairs of chunks of the feature rows)
constexpr int kDepthWeights = 4;    // and in the other products (2 measured 6 % slower, 8 the same)
constexpr int kRows = 64;           // rows per workgroup
constexpr int kThreads = 256;       // four wavefronts: 64 rows x 32 columns each of a 128-wide output
constexpr int kK1 = 384, kN1 = 128, kN2 = 128, kN3 = 64;
constexpr int kActStride = 136;     // 16-bit elements between rows of the activation planes: 128 + 8 (16-byte reads without bank conflicts)
constexpr int kKC = 16;             // k per staged chunk = one matrix instruction deep
constexpr int kStStride = 40;       // 16-bit elements between staged rows: a pair of chunks (32 k) + 8
constexpr int kParts = 2;           // half-precision parts per float32 operand
constexpr float kResidualScale = 2048.0f, kResidualBack = 1.0f / 2048.0f;      // 2^11

struct FusedArgs {
    const float* rows[4];           // [n_t, 384] feature rows per type
    int n[4];
    int tile_end[4];                // running sum of the per-type row tiles
    const float* w1t[4];            // [128, 384]: layer 1's weights, the summed index contiguous (transposed)
    const float* w2t[4];            // [128, 128]
    const float* w3t[4];            // [64, 128]
    const float* w1[4];             // [384, 128]: as stored -- the transposed operand of the way back
    const float* w2[4];             // [128, 128]
    const float* w3[4];             // [128, 64]
    const float* b1[4];
    const float* b2[4];
    const float* b3[4];
    const float* w4[4];             // [64]
    const float* b4[4];             // one float
    const float* scale[4];          // [n_t] gradient with respect to each row's value, or null (ones)
    float* value[4];                // [n_t]
    float* grad[4];                 // [n_t, 384], or null
    const unsigned short* packed;   // the six weight matrices of every type already split (pack_weights_kernel), or null
};

// Packed weights: per type the six matrices one after the other (layer 1 as stored as three matrices of 128 columns),
// each chunk by chunk of 16 k as [chunk][part][column][16 k] of half precision -- what a workgroup would otherwise split again
// for every tile of rows it takes, laid out so that a chunk's part is one contiguous run that the workgroup's
// threads copy 8 bytes each.
constexpr int kPackF1 = 0;                              // layer 1 transposed: 128 columns x 384
constexpr int kPackF2 = kPackF1 + kParts * kN1 * kK1;        // layer 2 transposed: 128 x 128
constexpr int kPackF3 = kPackF2 + kParts * kN2 * kN1;        // layer 3 transposed: 64 x 128
constexpr int kPackB1 = kPackF3 + kParts * kN3 * kN2;        // layer 1 as stored: 384 columns x 128
constexpr int kPackB2 = kPackB1 + kParts * kK1 * kN1;        // layer 2 as stored: 128 x 128
constexpr int kPackB3 = kPackB2 + kParts * kN1 * kN2;        // layer 3 as stored: 128 x 64
constexpr int kPackPerType = kPackB3 + kParts * kN2 * kN3;   // 294,912 half-precision values

struct __align__(16) FusedLds {
    union {
        unsigned short act[kParts][kRows][kActStride];        // a layer's activations or gradients, split: [part][row][k]
        unsigned short astage[2][kParts][kRows][kStStride];   // layer 1: pairs of chunks of the feature rows
    };
    float rowval[2][kRows];                              // the output layer's partial sums; then the rows' upstream factors
};

// two floats -> their two half-precision parts (the value rounded, and 2^11 times what the rounding left), each pair
// packed into one register (first value in the low half).  Both differences are exact in float32.
__device__ __forceinline__ void split_pair(float x0, float x1, unsigned& p1, unsigned& p2)
{
    const h2v h = __builtin_convertvector(f2v{x0, x1}, h2v);
    p1 = __builtin_bit_cast(unsigned, h);
    // 2^11 x - 2^11 h in one fused multiply-add that reads h as it is (both products are exact, and so is the difference)
    const float r0 = fmaf(static_cast<float>(h[0]), -kResidualScale, x0 * kResidualScale);
    const float r1 = fmaf(static_cast<float>(h[1]), -kResidualScale, x1 * kResidualScale);
    p2 = __builtin_bit_cast(unsigned, __builtin_convertvector(f2v{r0, r1}, h2v));
}

// a chunk piece (four consecutive k of one row or column) split into the planes of a stage buffer
template <int kR>
__device__ __forceinline__ void stage_piece(unsigned short (&dst)[kParts][kR][kStStride], int r, int k4, const v4 x)
{
    unsigned lo[kParts], hi[kParts];
    split_pair(x[0], x[1], lo[0], lo[1]);
    split_pair(x[2], x[3], hi[0], hi[1]);
#pragma unroll
    for (int q = 0; q < kParts; ++q) *reinterpret_cast<u2v*>(&dst[q][r][k4]) = u2v{lo[q], hi[q]};
}

__device__ __forceinline__ float celu_of(float v, float alpha, float inv_alpha)
{
    return v >= 0.f ? v : alpha * (__expf(v * inv_alpha) - 1.0f);
}
// CELU' from CELU's own value: 1 for h >= 0, exp(z / alpha) = h / alpha + 1 below
__device__ __forceinline__ float celu_slope(float h, float inv_alpha) { return h >= 0.f ? 1.0f : fmaf(h, inv_alpha, 1.0f); }

// sum over the 32 lanes of each half of the wavefront; lanes 16-31 and 48-63 hold the result
__device__ __forceinline__ float half_sum_to_upper_row(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));   // row_ror:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));   // row_ror:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));   // row_ror:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));   // row_ror:1
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));   // row_bcast:15
    return v;
}

// Positions.  A 128-wide output (kWide): the wavefront owns the tile's 64 rows x 32 columns, columns wave*32 + l32, as
// two 32 x 32 blocks one above the other -- block j, accumulator e is row j*32 + 8 (e / 4) + 4 half + e % 4.  The
// 64-wide output of layer 3: one block per wavefront, rows wr*32 + ..., columns wc*32 + l32.
struct Place {
    int tid, lane, wave, wr, wc, l32, half;
    __device__ __forceinline__ int rib(int e) const { return 8 * (e >> 2) + 4 * half + (e & 3); }      // row in the block
    template <bool kWide> __device__ __forceinline__ int row(int j, int e) const { return (kWide ? j * 32 : wr * 32) + rib(e); }
    template <bool kWide> __device__ __forceinline__ int col() const { return (kWide ? wave * 32 : wc * 32) + l32; }
};

// One layer's product for this workgroup's 64 rows: acc = A . B^T, A = 64 x kK (rows), B = (kWide ? 128 : 64) x kK
// (`wt`: one row per output column), chunk by chunk of 16 k.
// B never passes through LDS: a matrix instruction's operand is, per lane, eight consecutive k of one column -- 16
// bytes of a packed chunk, and the 64 lanes' pieces are one contiguous kilobyte -- so every wavefront loads its own
// operands straight into registers, kDepth chunks ahead.  In a 128-wide product a wavefront takes ALL 64 rows of 32
// columns: its weight operand serves two matrix instructions' worth of rows, no other wavefront loads the same
// columns, and the row operand -- from LDS, which has the bandwidth to spare -- is read twice as often instead.  (With
// 32 rows x 64 columns per wavefront the two wavefronts of a column half loaded the same weights: the weights' loads,
// 1.2 MB per tile through the compute unit's 64-byte-per-cycle load path, were the largest single part of the kernel.)
// With the weights staged in LDS (the first version) the kernel was bound by LDS traffic: nine kilobytes read and
// written per wavefront and chunk for six matrix instructions, and a barrier per chunk.  A comes from the activation
// planes, with no barrier inside the product; or (kAGlobal: layer 1) from `arows` in memory through a double-buffered
// LDS stage (the rows are float32 and have to be split and regrouped), one barrier per chunk.  Begins and ends with a
// barrier: the planes written before the call are complete, and afterwards nobody reads the planes or the stage any more.
// kPacked: `wt` points at the matrix's packed chunks (half precision); otherwise at float32 weights, of which a lane
// loads its eight values and splits them itself.
template <int kK, bool kWide, bool kAGlobal, bool kPacked, int kDepth>
__device__ __forceinline__ void layer_product(FusedLds& S, const Place& P, v16 (&acc)[2], const void* __restrict__ wt,
                                              const float* __restrict__ arows, int row0, int n)
{
    constexpr int chunks = kK / kKC;
    constexpr int kCols = kWide ? 128 : 64;              // output columns
    constexpr int kNB = kWide ? 2 : 1;                   // blocks (accumulators) of this wavefront
    static_assert(chunks % kDepth == 0 && kDepth >= 2, "the chunk loop is unrolled by the number of register sets");
    const int col = P.col<kWide>();
    // a chunk's weight operand for this wavefront's columns, as loaded: the two parts (packed), or eight float32 weights
    struct BSet {
        u4v raw[2];
    };
    BSet B[kDepth];
    auto bfetch = [&](int c, BSet& x) {
        if constexpr (kPacked) {
            const unsigned short* w = static_cast<const unsigned short*>(wt) + (c * kParts * kCols + col) * kKC + P.half * 8;
#pragma unroll
            for (int m = 0; m < kParts; ++m) x.raw[m] = *reinterpret_cast<const u4v*>(w + m * kCols * kKC);
        } else {
            const float* w = static_cast<const float*>(wt) + static_cast<size_t>(col) * kK + c * kKC + P.half * 8;
            x.raw[0] = *reinterpret_cast<const u4v*>(w);
            x.raw[1] = *reinterpret_cast<const u4v*>(w + 4);
        }
    };
    auto boperand = [&](const BSet& x, h8v (&bv)[kParts]) {
        if constexpr (kPacked) {
#pragma unroll
            for (int m = 0; m < kParts; ++m) bv[m] = __builtin_bit_cast(h8v, x.raw[m]);
        } else {
            u4v part[kParts];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const v4 f = __builtin_bit_cast(v4, x.raw[h]);
                unsigned a[kParts], b[kParts];
                split_pair(f[0], f[1], a[0], a[1]);
                split_pair(f[2], f[3], b[0], b[1]);
#pragma unroll
                for (int m = 0; m < kParts; ++m) {
                    part[m][2 * h] = a[m];
                    part[m][2 * h + 1] = b[m];
                }
            }
#pragma unroll
            for (int m = 0; m < kParts; ++m) bv[m] = __builtin_bit_cast(h8v, part[m]);
        }
    };
    // Layer 1: the feature rows go through LDS a PAIR of chunks (32 k = one 128-byte line per row) at a time: eight lanes
    // fetch a row's line together, a thread two rows' pieces (rows r8 and r8 + 32, k8..k8+3 of the pair), and a barrier
    // closes a pair, not a chunk.  kPairsAhead pairs are in flight in registers.
    constexpr int kPairsAhead = 2;
    static_assert(!kAGlobal || (kDepth == 2 * kPairsAhead && kRows == 64 && kThreads == 256), "the unrolled loop body is two pairs long");
    const int r8 = P.tid >> 3, k8 = (P.tid & 7) << 2;
    const int arow0 = min(row0 + r8, n - 1), arow1 = min(row0 + r8 + 32, n - 1);      // rows past the end: the last row again, never stored
    struct APair {
        v4 x[2];
    };
    APair A[kAGlobal ? kPairsAhead : 1];
    auto afetch = [&](int q, APair& a) {
        a.x[0] = *reinterpret_cast<const v4*>(arows + static_cast<size_t>(arow0) * kK + q * 2 * kKC + k8);
        a.x[1] = *reinterpret_cast<const v4*>(arows + static_cast<size_t>(arow1) * kK + q * 2 * kKC + k8);
    };
    auto astage_pair = [&](int q, const APair& a) {
        stage_piece(S.astage[q & 1], r8, k8, a.x[0]);
        stage_piece(S.astage[q & 1], r8 + 32, k8, a.x[1]);
    };

    v16 lo[2];                   // the mixed partial products, 2^11 times their size
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            acc[j][e] = 0.f;
            lo[j][e] = 0.f;
        }
#pragma unroll
    for (int s = 0; s < kDepth; ++s) bfetch(s, B[s]);
    if constexpr (kAGlobal) {
#pragma unroll
        for (int q = 0; q < kPairsAhead; ++q) afetch(q, A[q]);
        astage_pair(0, A[0]);
        if (2 * kPairsAhead < chunks) afetch(kPairsAhead, A[0]);
    }
    __syncthreads();             // pair 0 of the rows is staged; the activation planes written before this call are complete
    // chunk c: (layer 1, first chunk of a pair: stage the rows' next pair into the other buffer, ask for the pair
    // kPairsAhead further on,) multiply chunk c, ask for the weights of chunk c + kDepth
    auto step = [&](int c, BSet& b, APair& a_next) {
        h8v av[2][kParts];
#pragma unroll
        for (int j = 0; j < kNB; ++j) {
            const int arow_l = (kWide ? j * 32 : P.wr * 32) + P.l32;
#pragma unroll
            for (int m = 0; m < kParts; ++m) {
                if constexpr (kAGlobal)
                    av[j][m] = __builtin_bit_cast(h8v, *reinterpret_cast<const u4v*>(&S.astage[(c >> 1) & 1][m][arow_l][(c & 1) * kKC + P.half * 8]));
                else
                    av[j][m] = __builtin_bit_cast(h8v, *reinterpret_cast<const u4v*>(&S.act[m][arow_l][c * kKC + P.half * 8]));
            }
        }
        if constexpr (kAGlobal) {
            asm volatile("" ::: "memory");               // the reads above stay ahead of the stage's writes
            const int q = c >> 1;
            if ((c & 1) == 0 && 2 * (q + 1) < chunks) {
                astage_pair(q + 1, a_next);              // the other buffer: last read before the previous barrier
                if (2 * (q + 1 + kPairsAhead) < chunks) afetch(q + 1 + kPairsAhead, a_next);
            }
        }
        h8v bv[kParts];
        boperand(b, bv);
        // independent accumulators alternate, so that no matrix instruction waits for the one before it
#pragma unroll
        for (int j = 0; j < kNB; ++j) lo[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[j][1], bv[0], lo[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < kNB; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[j][0], bv[0], acc[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < kNB; ++j) lo[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[j][0], bv[1], lo[j], 0, 0, 0);
        if (c + kDepth < chunks) bfetch(c + kDepth, b);
        if constexpr (kAGlobal) {
            if (c & 1) __syncthreads();                  // the pair has been read, the next one is staged
        }
    };
    for (int c = 0; c < chunks; c += kDepth) {
        // (layer 1: kDepth = 2 kPairsAhead chunks; chunk c + u belongs to pair c / 2 + u / 2, and the pair staged during
        // it, one further on, sits in register set (u / 2 + 1) % kPairsAhead)
#pragma unroll
        for (int u = 0; u < kDepth; ++u) step(c + u, B[u], A[kAGlobal ? ((u >> 1) + 1) % kPairsAhead : 0]);
    }
    if constexpr (!kAGlobal) __syncthreads();
#pragma unroll
    for (int j = 0; j < kNB; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = fmaf(lo[j][e], kResidualBack, acc[j][e]);
}

// a wavefront's values of a layer -> the activation planes, split; column = k of the next product
template <bool kWide>
__device__ __forceinline__ void to_planes(FusedLds& S, const Place& P, const v16 (&v)[2])
{
    const int col = P.col<kWide>();
#pragma unroll
    for (int j = 0; j < (kWide ? 2 : 1); ++j) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
            unsigned p[kParts];
            split_pair(v[j][e], v[j][e + 1], p[0], p[1]);
            const int r0 = P.row<kWide>(j, e), r1 = P.row<kWide>(j, e + 1);
#pragma unroll
            for (int q = 0; q < kParts; ++q) {
                S.act[q][r0][col] = static_cast<unsigned short>(p[q] & 0xffffu);
                S.act[q][r1][col] = static_cast<unsigned short>(p[q] >> 16);
            }
        }
    }
}

template <bool kGrad, bool kPacked>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
void networks_fused_kernel(FusedArgs args, float alpha, float inv_alpha)
{
    static_assert(kRows == 64 && kThreads == 256, "four wavefronts: 64 rows x 32 columns each of a 128-wide output");
    __shared__ FusedLds S;
    Place P;
    P.tid = threadIdx.x;
    P.lane = P.tid & 63;
    P.wave = P.tid >> 6;
    P.wr = P.wave >> 1;
    P.wc = P.wave & 1;
    P.l32 = P.lane & 31;
    P.half = P.lane >> 5;
    const int tile = blockIdx.x;
    const int t = (tile >= args.tile_end[0]) + (tile >= args.tile_end[1]) + (tile >= args.tile_end[2]);
    const int first = t == 0 ? 0 : args.tile_end[t - 1];
    const int row0 = (tile - first) * kRows, n = args.n[t];

    // a layer's weights: split beforehand, or float32 as the caller holds them
    const unsigned short* const pk = kPacked ? args.packed + static_cast<size_t>(t) * kPackPerType : nullptr;
    auto weights = [&](const float* plain, int packed_at) -> const void* {
        if constexpr (kPacked) return pk + packed_at;
        else return plain;
    };
    const int cw = P.col<true>();                        // this lane's column of a 128-wide layer

    v16 acc[2], a1[2], a2[2], a3[2];
    // ------------------------------------------------------------ layer 1: 384 -> 128
    layer_product<kK1, true, true, kPacked, kDepthRows>(S, P, acc, weights(args.w1t[t], kPackF1), args.rows[t], row0, n);
    {
        const float b = args.b1[t][cw];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) a1[j][e] = celu_of(acc[j][e] + b, alpha, inv_alpha);
    }
    to_planes<true>(S, P, a1);
    // ------------------------------------------------------------ layer 2: 128 -> 128
    layer_product<kN1, true, false, kPacked, kDepthWeights>(S, P, acc, weights(args.w2t[t], kPackF2), nullptr, row0, n);
    {
        const float b = args.b2[t][cw];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) a2[j][e] = celu_of(acc[j][e] + b, alpha, inv_alpha);
    }
    to_planes<true>(S, P, a2);
    // ------------------------------------------------------------ layer 3: 128 -> 64, and the output layer 64 -> 1
    layer_product<kN2, false, false, kPacked, kDepthWeights>(S, P, acc, weights(args.w3t[t], kPackF3), nullptr, row0, n);
    const int c3 = P.col<false>();                       // this lane's column of the 64
    const float w4 = args.w4[t][c3];
    {
        const float b = args.b3[t][c3];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            a3[0][e] = celu_of(acc[0][e] + b, alpha, inv_alpha);
            const float tot = half_sum_to_upper_row(a3[0][e] * w4);      // over this wavefront's 32 of the 64 columns
            if (P.l32 == 16 + e) S.rowval[P.wc][P.row<false>(0, e)] = tot;
        }
    }
    __syncthreads();
    if (P.tid < kRows) {
        const int gr = row0 + P.tid;
        const float value = S.rowval[0][P.tid] + S.rowval[1][P.tid] + (args.b4[t] ? args.b4[t][0] : 0.f);
        if (gr < n) args.value[t][gr] = value;
    }
    if constexpr (!kGrad) return;
    // ------------------------------------------------------------ the way back
    __syncthreads();             // the partial sums have been read
    if (P.tid < kRows) S.rowval[0][P.tid] = args.scale[t] ? args.scale[t][min(row0 + P.tid, n - 1)] : 1.0f;
    __syncthreads();
    {
        v16 g3[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) g3[0][e] = w4 * celu_slope(a3[0][e], inv_alpha);     // for a unit upstream factor
        to_planes<false>(S, P, g3);
    }
    // g2 = (g3 W3^T) .* celu'(a2): 64 -> 128
    layer_product<kN3, true, false, kPacked, kDepthWeights>(S, P, acc, weights(args.w3[t], kPackB3), nullptr, row0, n);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] *= celu_slope(a2[j][e], inv_alpha);
    to_planes<true>(S, P, acc);
    // g1 = (g2 W2^T) .* celu'(a1): 128 -> 128
    layer_product<kN2, true, false, kPacked, kDepthWeights>(S, P, acc, weights(args.w2[t], kPackB2), nullptr, row0, n);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] *= celu_slope(a1[j][e], inv_alpha);
    to_planes<true>(S, P, acc);
    // dx = g1 W1^T: 128 -> 384, three column tiles of 128
    float* __restrict__ out = args.grad[t];
    float upstream[2][16];       // the upstream factors of this lane's rows
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) upstream[j][e] = S.rowval[0][P.row<true>(j, e)];
    for (int ct = 0; ct < kK1 / 128; ++ct) {
        const void* w;
        if constexpr (kPacked) w = pk + kPackB1 + static_cast<size_t>(ct) * kParts * 128 * kN1;
        else w = args.w1[t] + static_cast<size_t>(ct) * 128 * kN1;
        layer_product<kN1, true, false, kPacked, kDepthWeights>(S, P, acc, w, nullptr, row0, n);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int gr = row0 + P.row<true>(j, e);
                if (gr < n) out[static_cast<size_t>(gr) * kK1 + ct * 128 + cw] = acc[j][e] * upstream[j][e];
            }
        }
    }
}

// one float32 weight -> its two half-precision parts in the packed buffer; a thread per weight of one type's six matrices
__global__ __launch_bounds__(256) void pack_weights_kernel(FusedArgs args, unsigned short* __restrict__ packed)
{
    const int t = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;           // index among the type's 147,456 weights
    constexpr int n1 = kN1 * kK1, n2 = kN2 * kN1, n3 = kN3 * kN2;
    if (i >= 2 * (n1 + n2 + n3)) return;
    const float* src;
    int at, cols, k_len, j = i;      // the matrix: where it starts in the packed buffer, its columns and its summed length
    if (j < n1) { src = args.w1t[t]; at = kPackF1; cols = kN1; k_len = kK1; }
    else if ((j -= n1) < n2) { src = args.w2t[t]; at = kPackF2; cols = kN2; k_len = kN1; }
    else if ((j -= n2) < n3) { src = args.w3t[t]; at = kPackF3; cols = kN3; k_len = kN2; }
    else if ((j -= n3) < n1) {       // layer 1 as stored, [384][128]: three matrices of 128 columns
        src = args.w1[t];
        const int ct = j / (128 * kN1);
        src += ct * 128 * kN1;
        j -= ct * 128 * kN1;
        at = kPackB1 + ct * kParts * 128 * kN1;
        cols = 128;
        k_len = kN1;
    }
    else if ((j -= n1) < n2) { src = args.w2[t]; at = kPackB2; cols = kN1; k_len = kN2; }
    else { j -= n2; src = args.w3[t]; at = kPackB3; cols = kN2; k_len = kN3; }
    unsigned p1, p2;
    split_pair(src[j], 0.f, p1, p2);
    const int r = j / k_len, k = j - r * k_len;
    unsigned short* dst = packed + static_cast<size_t>(t) * kPackPerType + at + ((k / kKC) * kParts * cols + r) * kKC + (k % kKC);
    dst[0] = static_cast<unsigned short>(p1 & 0xffffu);
    dst[cols * kKC] = static_cast<unsigned short>(p2 & 0xffffu);
}

}  // namespace

size_t networks_packed_bytes() { return static_cast<size_t>(4) * kPackPerType * sizeof(unsigned short); }

// the six weight matrices of each type (three transposed, three as stored) split into `packed` (networks_packed_bytes())
hipError_t launch_networks_pack(const float* const w1t[4], const float* const w2t[4], const float* const w3t[4],
                                const float* const w1[4], const float* const w2[4], const float* const w3[4],
                                void* packed, hipStream_t stream)
{
    FusedArgs a = {};
    for (int t = 0; t < 4; ++t) {
        a.w1t[t] = w1t[t]; a.w2t[t] = w2t[t]; a.w3t[t] = w3t[t];
        a.w1[t] = w1[t]; a.w2[t] = w2[t]; a.w3[t] = w3[t];
    }
    constexpr int per_type = 2 * (kN1 * kK1 + kN2 * kN1 + kN3 * kN2);
    pack_weights_kernel<<<dim3((per_type + 255) / 256, 4), dim3(256), 0, stream>>>(a, static_cast<unsigned short*>(packed));
    return hipGetLastError();
}

// rows[t]: [n[t], 384]; w*t: transposed weights ([out, in]); w*: as stored ([in, out]); value[t]: [n[t]];
// grad[t]: [n[t], 384] or null pointers (then only the values are formed; w1, w2, w3 and scale are not read).
// packed: the weights as launch_networks_pack left them (then w*t and w* are not read), or null.
hipError_t launch_networks_fused(const float* const rows[4], const int32_t n[4],
                                 const float* const w1t[4], const float* const w2t[4], const float* const w3t[4],
                                 const float* const w1[4], const float* const w2[4], const float* const w3[4],
                                 const float* const b1[4], const float* const b2[4], const float* const b3[4],
                                 const float* const w4[4], const float* const b4[4], const float* const scale[4],
                                 float alpha, float* const value[4], float* const grad[4], const void* packed,
                                 hipStream_t stream)
{
    FusedArgs a = {};
    a.packed = static_cast<const unsigned short*>(packed);
    int tiles = 0;
    bool want_grad = false;
    for (int t = 0; t < 4; ++t) {
        a.rows[t] = rows[t];
        a.n[t] = n[t];
        tiles += (n[t] + kRows - 1) / kRows;
        a.tile_end[t] = tiles;
        a.w1t[t] = w1t ? w1t[t] : nullptr; a.w2t[t] = w2t ? w2t[t] : nullptr; a.w3t[t] = w3t ? w3t[t] : nullptr;
        a.w1[t] = w1 ? w1[t] : nullptr; a.w2[t] = w2 ? w2[t] : nullptr; a.w3[t] = w3 ? w3[t] : nullptr;
        a.b1[t] = b1[t]; a.b2[t] = b2[t]; a.b3[t] = b3[t];
        a.w4[t] = w4[t];
        a.b4[t] = b4 ? b4[t] : nullptr;
        a.scale[t] = scale ? scale[t] : nullptr;
        a.value[t] = value[t];
        a.grad[t] = grad ? grad[t] : nullptr;
        want_grad = want_grad || (grad && grad[t]);
    }
    if (tiles == 0) return hipSuccess;
    const dim3 grid(static_cast<unsigned>(tiles)), block(kThreads);
    if (want_grad) {
        if (packed) networks_fused_kernel<true, true><<<grid, block, 0, stream>>>(a, alpha, 1.0f / alpha);
        else networks_fused_kernel<true, false><<<grid, block, 0, stream>>>(a, alpha, 1.0f / alpha);
    } else {
        if (packed) networks_fused_kernel<false, true><<<grid, block, 0, stream>>>(a, alpha, 1.0f / alpha);
        else networks_fused_kernel<false, false><<<grid, block, 0, stream>>>(a, alpha, 1.0f / alpha);
    }
    return hipGetLastError();
}

}  // namespace khan
