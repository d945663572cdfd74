// First dense layer of the per-type atomic networks, right behind the featurizer:
//     out[r, :] = act(rows[r, :] . W + b),   rows [n, 384] feature rows of one atom type, W [384, 128], b [128]
// (reference: khan/model/nn.py:38-68 -- tf.matmul + bias + activation per type -- with the CELU of
// khan/model/activations.py:63-65 as activation, or none).  float32 in, float32 accumulation on the matrix cores
// (v_mfma_f32_32x32x2_f32): the same arithmetic as a float32 matrix product, in another summation order.
//
// One workgroup of four wavefronts owns a 128-row x 128-column tile of the output of one type; every wavefront a
// 64 x 64 quarter of it = 2 x 2 matrix-core blocks of 32 x 32, whose 64 accumulator registers stay in the lanes
// for the whole K = 384 loop.  K is walked in chunks of 32: a chunk of the rows (128 x 32) and of the transposed
// weights (128 x 32) is staged in LDS through registers, double buffered, so the global loads of chunk c+1 are in
// flight while chunk c is multiplied.  In LDS both tiles are [row or column][k] with the k run padded from 32 to 36
// floats: a lane reads four consecutive k of its row with one 16-byte read, conflict-free.  A matrix-core step
// multiplies two k per block: the lower half of the wavefront supplies k = 8q + t, the upper half k = 8q + 4 + t
// (t = 0..3 from one 16-byte read each), which covers every k of the chunk once -- a sum does not care about its order.
// The four types are one launch: a workgroup finds its type and tile from the per-type tile counts.
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

namespace {

constexpr int kDenseIn = kFeats;       // 384
constexpr int kDenseOut = 128;
constexpr int kTileRows = 128;
constexpr int kChunk = 32;             // k per staging step
constexpr int kPad = 36;               // floats per staged row: 32 + 4 (bank rotation for 16-byte reads)

typedef float v4 __attribute__((ext_vector_type(4)));
typedef float v16 __attribute__((ext_vector_type(16)));

struct DenseArgs {
    const float* rows[4];      // [n_t, 384] per type
    const float* wt[4];        // [128, 384]: the layer's weights transposed (k contiguous)
    const float* bias[4];      // [128]
    float* out[4];             // [n_t, 128]
    int n[4];                  // rows per type
    int tile_end[4];           // running sum of the per-type tile counts
};

struct __align__(16) DenseLds {
    float a[2][kTileRows][kPad];       // rows tile, double buffered
    float b[2][kDenseOut][kPad];       // transposed-weights tile
};

template <bool kCelu>
__global__ __launch_bounds__(256) void dense_first_kernel(DenseArgs args, float alpha, float inv_alpha)
{
    __shared__ DenseLds S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // type and tile of this workgroup
    const int blk = blockIdx.x;
    const int t = (blk >= args.tile_end[0]) + (blk >= args.tile_end[1]) + (blk >= args.tile_end[2]);
    const int tile = blk - (t == 0 ? 0 : args.tile_end[t - 1]);
    const int n = args.n[t];
    const float* __restrict__ rows = args.rows[t];
    const float* __restrict__ wt = args.wt[t];
    const int row0 = tile * kTileRows;

    // staging: a chunk of each tile is 128 x 32 floats = 1,024 pieces of 16 bytes, four per thread:
    // piece p = tid + 256 u -> tile row p / 8, k offset (p % 8) * 4
    v4 ra[4], rb[4];
    auto fetch = [&](int chunk) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int p = tid + 256 * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            const int gr = row0 + r;
            ra[u] = v4{0.f, 0.f, 0.f, 0.f};
            if (gr < n) ra[u] = *reinterpret_cast<const v4*>(rows + static_cast<size_t>(gr) * kDenseIn + chunk * kChunk + k4);
            rb[u] = *reinterpret_cast<const v4*>(wt + static_cast<size_t>(r) * kDenseIn + chunk * kChunk + k4);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int p = tid + 256 * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            *reinterpret_cast<v4*>(&S.a[buf][r][k4]) = ra[u];
            *reinterpret_cast<v4*>(&S.b[buf][r][k4]) = rb[u];
        }
    };

    // this wavefront's 64 x 64 quarter: rows wr*64.., columns wc*64..; two blocks of 32 each way
    const int wr = wave >> 1, wc = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;
    v16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    constexpr int kChunks = kDenseIn / kChunk;      // 12
    fetch(0);
    stage(0);
    __syncthreads();
    for (int c = 0; c < kChunks; ++c) {
        const int buf = c & 1;
        if (c + 1 < kChunks) fetch(c + 1);          // in flight while this chunk is multiplied
#pragma unroll
        for (int q = 0; q < kChunk / 8; ++q) {
            // four consecutive k of this lane's row / column: k = 8q + 4 half + (0..3)
            v4 av[2], bv[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) av[i] = *reinterpret_cast<const v4*>(&S.a[buf][wr * 64 + i * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bv[j] = *reinterpret_cast<const v4*>(&S.b[buf][wc * 64 + j * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
        }
        if (c + 1 < kChunks) {
            stage(buf ^ 1);                          // the other buffer: nobody reads it during this chunk
            __syncthreads();
        }
    }

    // epilogue: bias, activation, store.  Accumulator e of block (i, j) is output row
    // wr*64 + i*32 + 8 (e / 4) + 4 half + e % 4, column wc*64 + j*32 + l32.
    const float* __restrict__ bias = args.bias[t];
    float* __restrict__ out = args.out[t];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = wc * 64 + j * 32 + l32;
        const float bj = bias[col];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int r = row0 + wr * 64 + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                float v = acc[i][j][e] + bj;
                if (kCelu) v = v >= 0.f ? v : alpha * (__expf(v * inv_alpha) - 1.0f);
                if (r < n) out[static_cast<size_t>(r) * kDenseOut + col] = v;
            }
        }
    }
}

}  // namespace

hipError_t launch_dense_first(const float* const rows[4], const int32_t n[4], const float* const wt[4],
                              const float* const bias[4], bool celu, float alpha, float* const out[4],
                              hipStream_t stream)
{
    DenseArgs a;
    int run = 0;
    for (int t = 0; t < 4; ++t) {
        a.rows[t] = rows[t];
        a.wt[t] = wt[t];
        a.bias[t] = bias[t];
        a.out[t] = out[t];
        a.n[t] = n[t];
        run += (n[t] + kTileRows - 1) / kTileRows;
        a.tile_end[t] = run;
    }
    if (run == 0) return hipSuccess;
    if (celu) dense_first_kernel<true><<<dim3(static_cast<unsigned>(run)), dim3(256), 0, stream>>>(a, alpha, 1.0f / alpha);
    else dense_first_kernel<false><<<dim3(static_cast<unsigned>(run)), dim3(256), 0, stream>>>(a, alpha, 1.0f);
    return hipGetLastError();
}

}  // namespace khan
