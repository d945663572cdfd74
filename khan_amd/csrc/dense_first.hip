// Dense layers of the per-type atomic networks on the matrix cores:
//     out[r, :] = act(in'[r, :] . W + b),   in' = in, or in .* CELU'(value) taken from a layer's own activations,
// for the four atom types in one launch (reference: khan/model/nn.py:38-68 -- tf.matmul + bias + activation per
// type -- with the CELU of khan/model/activations.py:63-65 as activation, or none).  The first form is a layer's
// forward pass (the first layer right behind the featurizer: in = the 384-wide feature rows); the second is the data
// gradient of a layer on the way back (in = the gradient with respect to the layer's activations, W = the layer's
// weights read the other way round, no bias, no activation).  float32 in, float32 accumulation: the arithmetic of a
// float32 matrix product, in another summation order.  Two forms of the products: on the float32 matrix instructions
// (v_mfma_f32_32x32x2_f32; dense_kernel and dense_pipe_kernel, described first), and -- the default -- on the bfloat16
// matrix instructions with every float32 operand split exactly into three bfloat16 parts (dense_split_kernel, further
// down), which gives the same result to float32 accuracy in less than half the matrix time.
//
// One workgroup of four wavefronts owns a tile of 128 rows x kTileCols columns of the output of one type.  With 128
// columns every wavefront has a 64 x 64 quarter of it = 2 x 2 matrix-core blocks of 32 x 32; with 64 columns (the third
// layer's width) a 32 x 64 strip = 1 x 2 blocks.  The accumulators stay in the lanes for the whole K loop.  K is
// walked in chunks of 32: a chunk of the rows (128 x 32) and of the transposed weights (kTileCols x 32) is staged in LDS
// through registers, double buffered, so the global loads of chunk c+1 are in flight while chunk c is multiplied; the
// multiplication by the activation's derivative happens in those registers.  In LDS both tiles are [row or column][k]
// with the k run padded from 32 to 36 floats: a lane reads four consecutive k of its row with one 16-byte read,
// conflict-free.  A matrix-core step multiplies two k per block: the lower half of the wavefront supplies k = 8q + t,
// the upper half k = 8q + 4 + t (t = 0..3 from one 16-byte read each), which covers every k of the chunk once -- a
// sum does not care about its order.  A workgroup finds its type, row tile and column tile from the per-type tile
// counts; the column tiles of one row tile are neighbours in the grid, so the rows they share come from L2.
//
// Two extras fold the networks' output layer (n -> 1, no activation: nn.py:38-68 with the last entry of the layer
// sizes) into its neighbour.  kHead (64-column tile): the epilogue also forms head_out[r] = out[r, :] . head_w + head_b,
// a sum over the tile's 64 columns = over the 32 lanes that hold a row's values.  kRank1: on the way back the
// gradient with respect to the last hidden layer's activations is the outer product scale[r] * head_w[c]; the
// staging builds it in registers instead of reading a matrix that something else would have had to write.
#include <cstdlib>
#include <cstring>
#include "khan_internal.h"
#include "khan_params.h"

namespace khan {

namespace {

constexpr int kTileRows = 128;
constexpr int kChunk = 32;             // k per staging step
constexpr int kPad = 36;               // floats per staged row: 32 + 4 (bank rotation for 16-byte reads)

typedef float v4 __attribute__((ext_vector_type(4)));
typedef float v16 __attribute__((ext_vector_type(16)));

struct DenseArgs {
    const float* rows[4];      // [n_t, k] per type
    const float* deriv[4];     // [n_t, k] activations whose CELU derivative multiplies the rows, or null
    const float* wt[4];        // [n_out, k]: the weights with the summed index contiguous
    const float* bias[4];      // [n_out], or null
    float* out[4];             // [n_t, n_out]
    int n[4];                  // rows per type
    int tile_end[4];           // running sum of the per-type (row tile x column tile) counts
    int k, n_out, col_tiles;
    const float* head_w[4];    // kHead: [n_out] weights of the output layer; kRank1: [k], the same weights on the way back
    const float* head_b[4];    // kHead: one float, or null
    float* head_out[4];        // kHead: [n_t]
    const float* scale[4];     // kRank1: [n_t], the gradient with respect to each row's output value
};

// sum over the 32 lanes of each half of the wavefront; lanes 16-31 and 48-63 hold the result
__device__ __forceinline__ float half_sum_to_upper_row(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));   // row_ror:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));   // row_ror:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));   // row_ror:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));   // row_ror:1
    // rows 1 and 3 add lane 15 of the row before them (rows 0 and 2 add the zero given as old value)
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xa, 0xf, false));   // row_bcast:15
    return v;
}

// Rows of a staging piece built from the outer product scale[row] * head_w[k..k+3]
__device__ __forceinline__ v4 rank1_piece(const float* __restrict__ scale, const float* __restrict__ head_w, int row, int k)
{
    const float sc = scale[row];
    const v4 w = *reinterpret_cast<const v4*>(head_w + k);
    return v4{sc * w[0], sc * w[1], sc * w[2], sc * w[3]};
}

// Epilogue of one tile for one wavefront: bias, activation, store; with kHead (one wavefront holds all 64 columns of
// its 32 rows) also the output layer's value of every row.  Accumulator e of block (i, j) is output row
// row_base + i*32 + 8 (e / 4) + 4 half + e % 4, column col_base + j*32 + l32.
// The bias is waited for once, before the first store: a wait inside a conditional store would also wait for
// the stores before it (loads and stores share one counter), one by one -- 64 stores, each at full latency.
template <bool kCelu, bool kHead, int kBI>
__device__ __forceinline__ void tile_epilogue(const v16 (&acc)[kBI][2], float (&bj)[2], float (&hw)[2], const float* head_b,
                                              float* __restrict__ out, float* __restrict__ head_out, int n, int n_out,
                                              int row_base, int col_base, int l32, int half, float alpha, float inv_alpha)
{
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        asm volatile("" : "+v"(bj[j]));          // in its register from here on: the one wait happens here
        if constexpr (kHead) asm volatile("" : "+v"(hw[j]));
    }
    float hb = 0.f;
    if constexpr (kHead) {
        hb = head_b ? *head_b : 0.f;
        asm volatile("" : "+v"(hb));
    }
#pragma unroll
    for (int i = 0; i < kBI; ++i) {
        float dot[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) dot[e] = 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = col_base + j * 32 + l32;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int r = row_base + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                float v = acc[i][j][e] + bj[j];
                if (kCelu) v = v >= 0.f ? v : alpha * (__expf(v * inv_alpha) - 1.0f);
                if (r < n) out[static_cast<size_t>(r) * n_out + col] = v;
                if constexpr (kHead) dot[e] = fmaf(v, hw[j], dot[e]);
            }
        }
        if constexpr (kHead) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float tot = half_sum_to_upper_row(dot[e]) + hb;
                const int r = row_base + i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
                if (l32 == 16 + e && r < n) head_out[r] = tot;        // lane 16 + e of each half stores row e's value
            }
        }
    }
}


template <int kTileCols>
struct __align__(16) DenseLds {
    float a[2][kTileRows][kPad];       // rows tile, double buffered
    float b[2][kTileCols][kPad];       // transposed-weights tile
};

// The plain form, one tile per workgroup, for any summed width that is a multiple of 32 (the widths of the
// reference's default network take the pipelined kernel below).
template <int kTileCols, bool kCelu, bool kDeriv, bool kHead, bool kRank1>
__global__ __launch_bounds__(256) void dense_kernel(DenseArgs args, float alpha, float inv_alpha)
{
    static_assert(!kHead || kTileCols == 64, "the output layer's sum runs over one wavefront's 64 columns");
    constexpr int kWaveRows = kTileCols == 128 ? 64 : 32;      // rows of a wavefront's part of the tile
    constexpr int kBI = kWaveRows / 32;                        // its matrix-core blocks down (2 or 1); across: 2
    constexpr int kBPieces = kTileCols * (kChunk / 4) / 256;   // 16-byte pieces of the weight chunk per thread (4 or 2)
    __shared__ DenseLds<kTileCols> S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // type, row tile and column tile of this workgroup
    const int blk = blockIdx.x;
    const int t = (blk >= args.tile_end[0]) + (blk >= args.tile_end[1]) + (blk >= args.tile_end[2]);
    const int rel = blk - (t == 0 ? 0 : args.tile_end[t - 1]);
    const int tile = rel / args.col_tiles, ctile = rel - tile * args.col_tiles;
    const int n = args.n[t], K = args.k;
    const float* __restrict__ rows = args.rows[t];
    const float* __restrict__ deriv = args.deriv[t];
    const float* __restrict__ wt = args.wt[t] + static_cast<size_t>(ctile) * kTileCols * K;
    const int row0 = tile * kTileRows, col0 = ctile * kTileCols;

    // staging: a chunk of the rows tile is 128 x 32 floats = 1,024 pieces of 16 bytes, four per thread:
    // piece p = tid + 256 u -> tile row p / 8, k offset (p % 8) * 4; the weight chunk likewise (kTileCols rows)
    v4 ra[4], rb[kBPieces];
    auto fetch = [&](int chunk) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int p = tid + 256 * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            // rows past the end of the type read its last row: their products are never stored, and a load that is
            // not under a condition needs no merge with a default afterwards (which would wait for it on the spot)
            const int gr = min(row0 + r, n - 1);
            const size_t at = static_cast<size_t>(gr) * K + chunk * kChunk + k4;
            if constexpr (kRank1) ra[u] = rank1_piece(args.scale[t], args.head_w[t], gr, chunk * kChunk + k4);
            else ra[u] = *reinterpret_cast<const v4*>(rows + at);
            if constexpr (kDeriv) {
                // CELU'(z) from CELU(z) = h: 1 for h >= 0, exp(z / alpha) = h / alpha + 1 below
                const v4 h = *reinterpret_cast<const v4*>(deriv + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) ra[u][e] *= h[e] >= 0.f ? 1.0f : fmaf(h[e], inv_alpha, 1.0f);
            }
        }
#pragma unroll
        for (int u = 0; u < kBPieces; ++u) {
            const int p = tid + 256 * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            rb[u] = *reinterpret_cast<const v4*>(wt + static_cast<size_t>(r) * K + chunk * kChunk + k4);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int p = tid + 256 * u;
            *reinterpret_cast<v4*>(&S.a[buf][p >> 3][(p & 7) << 2]) = ra[u];
        }
#pragma unroll
        for (int u = 0; u < kBPieces; ++u) {
            const int p = tid + 256 * u;
            *reinterpret_cast<v4*>(&S.b[buf][p >> 3][(p & 7) << 2]) = rb[u];
        }
    };

    // this wavefront's part: 128 columns -> rows wr*64.., columns wc*64..; 64 columns -> rows wave*32.., all columns
    const int wr = kTileCols == 128 ? (wave >> 1) : wave, wc = kTileCols == 128 ? (wave & 1) : 0;
    const int l32 = lane & 31, half = lane >> 5;
    v16 acc[kBI][2];
#pragma unroll
    for (int i = 0; i < kBI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int chunks = K / kChunk;
    fetch(0);
    stage(0);
    __syncthreads();
    for (int c = 0; c < chunks; ++c) {
        const int buf = c & 1;
        if (c + 1 < chunks) fetch(c + 1);          // in flight while this chunk is multiplied
#pragma unroll
        for (int q = 0; q < kChunk / 8; ++q) {
            // four consecutive k of this lane's row / column: k = 8q + 4 half + (0..3)
            v4 av[kBI], bv[2];
#pragma unroll
            for (int i = 0; i < kBI; ++i) av[i] = *reinterpret_cast<const v4*>(&S.a[buf][wr * kWaveRows + i * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bv[j] = *reinterpret_cast<const v4*>(&S.b[buf][wc * 64 + j * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < kBI; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
        }
        if (c + 1 < chunks) {
            stage(buf ^ 1);                          // the other buffer: nobody reads it during this chunk
            __syncthreads();
        }
    }

    const float* __restrict__ bias = args.bias[t];
    float bj[2], hw[2] = {0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        bj[j] = bias ? bias[col0 + wc * 64 + j * 32 + l32] : 0.f;
        if constexpr (kHead) hw[j] = args.head_w[t][col0 + j * 32 + l32];
    }
    tile_epilogue<kCelu, kHead, kBI>(acc, bj, hw, args.head_b[t], args.out[t], args.head_out[t], n, args.n_out,
                                     row0 + wr * kWaveRows, col0 + wc * 64, l32, half, alpha, inv_alpha);
}

// The same product for the network's own widths (kK = 384, 128 or 64: an even number of chunks), as a pipeline that
// does not drain between tiles.  The grid is as many workgroups as stay resident; a workgroup takes tiles blk,
// blk + grid, ... and walks their chunks as one sequence of steps.  At step s it issues the global loads of step s + 2
// into one of two register sets, multiplies step s out of LDS, then stages the registers of step s + 1 -- loaded a
// whole step ago -- into the other LDS buffer.  So the first chunk of the next tile arrives while this tile is still
// being multiplied, and its epilogue's stores drain under the next tile's products: with K = 128 a tile is only four
// chunks long, and starting every tile cold cost a third of the kernel.
// kThreads: 512 for the 128-column tile (eight wavefronts, 4 down x 2 across, 32 x 64 each; two workgroups per CU are
// four wavefronts per SIMD, which need 128 registers or fewer), 256 for the 64-column tile (four wavefronts, 4 x 1).
template <int kTileCols, int kThreads, int kK, bool kCelu, bool kDeriv, bool kHead, bool kRank1>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(kThreads / 128, kThreads / 128)))
void dense_pipe_kernel(DenseArgs args, int total_tiles, float alpha, float inv_alpha)
{
    static_assert(!kHead || kTileCols == 64, "the output layer's sum runs over one wavefront's 64 columns");
    constexpr int kAcross = kTileCols / 64;                    // wavefronts across the tile
    constexpr int kWaveRows = kTileRows / (kThreads / 64 / kAcross);
    static_assert(kWaveRows == 32, "one 32-row block down, two across per wavefront");
    constexpr int kBI = kWaveRows / 32;
    constexpr int kAPieces = kTileRows * (kChunk / 4) / kThreads;    // 16-byte pieces of the rows chunk per thread
    constexpr int kBPieces = kTileCols * (kChunk / 4) / kThreads;    // and of the weight chunk
    constexpr int kChunks = kK / kChunk;
    static_assert(kChunks % 2 == 0, "two register sets alternate by step: a tile must be an even number of steps");
    __shared__ DenseLds<kTileCols> S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int stride = gridDim.x;

    struct Cursor {                 // where the next loads come from: a tile (or none) and a chunk of it
        const float* rows;          // kRank1: the per-row factors
        const float* head_w;
        const float* deriv;
        const float* wt;
        int row0, n, chunk, tile;
        bool live;
    };
    struct TileOut {                // what the epilogue of a tile needs
        float* out;
        float* head_out;
        const float* head_b;
        int row0, col0, n;
        float bj[2];                // the bias of this lane's two columns, loaded when the tile starts
        float hw[2];                // kHead: the output layer's weights of those columns
    };
    auto decode_loads = [&](int id, Cursor& c) {
        const int t = (id >= args.tile_end[0]) + (id >= args.tile_end[1]) + (id >= args.tile_end[2]);
        const int rel = id - (t == 0 ? 0 : args.tile_end[t - 1]);
        const int tile = rel / args.col_tiles, ctile = rel - tile * args.col_tiles;
        c.rows = kRank1 ? args.scale[t] : args.rows[t];
        c.head_w = args.head_w[t];
        c.deriv = args.deriv[t];
        c.wt = args.wt[t] + static_cast<size_t>(ctile) * kTileCols * kK;
        c.row0 = tile * kTileRows;
        c.n = args.n[t];
    };
    auto decode_out = [&](int id, TileOut& o) {
        const int t = (id >= args.tile_end[0]) + (id >= args.tile_end[1]) + (id >= args.tile_end[2]);
        const int rel = id - (t == 0 ? 0 : args.tile_end[t - 1]);
        const int tile = rel / args.col_tiles, ctile = rel - tile * args.col_tiles;
        o.out = args.out[t];
        o.row0 = tile * kTileRows;
        o.col0 = ctile * kTileCols;
        o.n = args.n[t];
        const float* bias = args.bias[t];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            o.bj[j] = bias ? bias[o.col0 + (kAcross == 2 ? (wave & 1) : 0) * 64 + j * 32 + (lane & 31)] : 0.f;
            o.hw[j] = 0.f;
            if constexpr (kHead) o.hw[j] = args.head_w[t][o.col0 + j * 32 + (lane & 31)];
        }
        o.head_out = args.head_out[t];
        o.head_b = args.head_b[t];
    };

    v4 ra[2][kAPieces], rb[2][kBPieces];
    auto fetch = [&](const Cursor& c, v4 (&a)[kAPieces], v4 (&b)[kBPieces]) {
        if (!c.live) return;
#pragma unroll
        for (int u = 0; u < kAPieces; ++u) {
            const int p = tid + kThreads * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            const int gr = min(c.row0 + r, c.n - 1);       // past the end: the last row again, never stored
            const size_t at = static_cast<size_t>(gr) * kK + c.chunk * kChunk + k4;
            if constexpr (kRank1) a[u] = rank1_piece(c.rows, c.head_w, gr, c.chunk * kChunk + k4);
            else a[u] = *reinterpret_cast<const v4*>(c.rows + at);
            if constexpr (kDeriv) {
                const v4 h = *reinterpret_cast<const v4*>(c.deriv + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) a[u][e] *= h[e] >= 0.f ? 1.0f : fmaf(h[e], inv_alpha, 1.0f);
            }
        }
#pragma unroll
        for (int u = 0; u < kBPieces; ++u) {
            const int p = tid + kThreads * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            b[u] = *reinterpret_cast<const v4*>(c.wt + static_cast<size_t>(r) * kK + c.chunk * kChunk + k4);
        }
    };
    auto stage = [&](int buf, const v4 (&a)[kAPieces], const v4 (&b)[kBPieces]) {
#pragma unroll
        for (int u = 0; u < kAPieces; ++u) {
            const int p = tid + kThreads * u;
            *reinterpret_cast<v4*>(&S.a[buf][p >> 3][(p & 7) << 2]) = a[u];
        }
#pragma unroll
        for (int u = 0; u < kBPieces; ++u) {
            const int p = tid + kThreads * u;
            *reinterpret_cast<v4*>(&S.b[buf][p >> 3][(p & 7) << 2]) = b[u];
        }
    };

    const int wr = kAcross == 2 ? (wave >> 1) : wave, wc = kAcross == 2 ? (wave & 1) : 0;
    const int l32 = lane & 31, half = lane >> 5;
    v16 acc[kBI][2];
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < kBI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int q = 0; q < kChunk / 8; ++q) {
            v4 av[kBI], bv[2];
#pragma unroll
            for (int i = 0; i < kBI; ++i) av[i] = *reinterpret_cast<const v4*>(&S.a[buf][wr * kWaveRows + i * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bv[j] = *reinterpret_cast<const v4*>(&S.b[buf][wc * 64 + j * 32 + l32][q * 8 + half * 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < kBI; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i][e], bv[j][e], acc[i][j], 0, 0, 0);
        }
    };
    auto epilogue = [&](TileOut& o) {
        tile_epilogue<kCelu, kHead, kBI>(acc, o.bj, o.hw, o.head_b, o.out, o.head_out, o.n, args.n_out,
                                         o.row0 + wr * kWaveRows, o.col0 + wc * 64, l32, half, alpha, inv_alpha);
    };

    // the load cursor runs two steps ahead of the multiplication
    Cursor cu;
    cu.tile = blockIdx.x;
    cu.chunk = 0;
    cu.live = cu.tile < total_tiles;
    if (!cu.live) return;
    decode_loads(cu.tile, cu);
    auto advance = [&]() {          // one step further
        if (++cu.chunk == kChunks) {
            cu.chunk = 0;
            cu.tile += stride;
            cu.live = cu.tile < total_tiles;
            if (cu.live) decode_loads(cu.tile, cu);
        }
    };
    // prologue: step 0 into LDS buffer 0, step 1 into register set 1
    fetch(cu, ra[0], rb[0]);
    advance();
    fetch(cu, ra[1], rb[1]);
    advance();
    stage(0, ra[0], rb[0]);
    __syncthreads();
    clear();
    for (int tile = blockIdx.x; tile < total_tiles; tile += stride) {
        const bool more = tile + stride < total_tiles;
        TileOut cur;
        decode_out(tile, cur);
        for (int c = 0; c < kChunks; c += 2) {
            // even step: LDS buffer 0 is multiplied, set 0 loads two steps ahead, set 1 (one step ahead) is staged
            fetch(cu, ra[0], rb[0]);
            advance();
            multiply(0);
            stage(1, ra[1], rb[1]);
            __syncthreads();
            // odd step
            fetch(cu, ra[1], rb[1]);
            advance();
            multiply(1);
            if (c + 2 < kChunks || more) {           // something follows: the first chunk of the next tile, at a tile's end
                stage(0, ra[0], rb[0]);
                __syncthreads();
            }
        }
        epilogue(cur);
        clear();
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same float32 product on the bfloat16 matrix instructions, which run sixteen times as fast as the float32 ones.
// Every float32 operand is split exactly into three bfloat16 values, x = x1 + x2 + x3 (8 + 8 + 8 significant bits:
// x1 = bf16(x), x2 = bf16(x - x1), x3 = bf16(x - x1 - x2); both differences are exact in float32), and of the nine
// partial products of x w the six largest are formed, each an exact 16-bit product accumulated in float32:
//     x w ~ x1 w1 + x1 w2 + x2 w1 + x2 w2 + x1 w3 + x3 w1.
// What is left out (x2 w3 + x3 w2 + x3 w3) is below 2^-23 |x w| (measured: 3e-9 of sum |x| |w| on a 384-term sum, against
// 3e-7 for the rounding of the float32 accumulation itself), so the result is a float32 matrix product to float32
// accuracy: six matrix instructions of 32 x 32 x 16 in place of eight of 32 x 32 x 2, at 32 instead of 64 cycles each.
// The splitting happens while a chunk is staged (rows: after the activation's derivative has been multiplied in; the
// weights likewise, in every workgroup: no second copy of the weights has to be kept).  In LDS a chunk is three planes
// of [row or column][32 k] bfloat16, rows 80 bytes apart (16-byte reads without bank conflicts).
// Eight wavefronts (128 columns) or four (64 columns) per workgroup, 32 rows x 64 columns each; one LDS buffer: the next
// chunk's global loads are in flight during the products, and the workgroups that share a CU alternate.
constexpr int kSplitStride = 40;       // bfloat16 elements between staged rows: 32 + 8

typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f2v __attribute__((ext_vector_type(2)));

template <int kTileCols, int kCT>
struct __align__(16) SplitLds {
    unsigned short a[3][kTileRows][kSplitStride];
    unsigned short b[kCT][3][kTileCols][kSplitStride];
};

// two floats -> their three bfloat16 parts, each pair packed into one register (first value in the low half)
__device__ __forceinline__ void split_pair(float x0, float x1, unsigned& p1, unsigned& p2, unsigned& p3)
{
    p1 = __builtin_bit_cast(unsigned, __builtin_convertvector(f2v{x0, x1}, bf16x2));
    const float r0 = x0 - __uint_as_float(p1 << 16), r1 = x1 - __uint_as_float(p1 & 0xffff0000u);
    p2 = __builtin_bit_cast(unsigned, __builtin_convertvector(f2v{r0, r1}, bf16x2));
    const float s0 = r0 - __uint_as_float(p2 << 16), s1 = r1 - __uint_as_float(p2 & 0xffff0000u);
    p3 = __builtin_bit_cast(unsigned, __builtin_convertvector(f2v{s0, s1}, bf16x2));
}

// kCT: column tiles that one workgroup multiplies at once (1, or all 3 of a 384-wide output: the rows are then staged
// and split once for the three, a step holds three times the products between its barriers, and one workgroup of eight
// wavefronts fills a CU -- 120 KB of LDS, 96 accumulator registers per lane).
template <int kTileCols, bool kCelu, bool kDeriv, bool kHead, bool kRank1, int kCT = 1>
__global__ __launch_bounds__(kTileCols * 4) void dense_split_kernel(DenseArgs args, int row_tiles, float alpha, float inv_alpha)
{
    static_assert(!kHead || kTileCols == 64, "the output layer's sum runs over one wavefront's 64 columns");
    constexpr int kThreads = kTileCols * 4;                          // 512 or 256: one wavefront per 32 rows x 64 columns
    constexpr int kAPieces = kTileRows * (kChunk / 4) / kThreads;    // 16-byte pieces of the rows chunk per thread (2 or 4)
    constexpr int kBPieces = kTileCols * (kChunk / 4) / kThreads;    // and of the weight chunk (2)
    static_assert(kCT == 1 || (kTileCols == 128 && !kHead), "several column tiles at once: 128-column tiles, no output layer");
    __shared__ SplitLds<kTileCols, kCT> S;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = args.k, chunks = K / kChunk, col_tiles = args.col_tiles / kCT;     // column tiles as the workgroups see them
    // row tiles of the four types, counted through: tile_end holds (row tiles x column tiles) sums
    const int rt_end0 = args.tile_end[0] / args.col_tiles, rt_end1 = args.tile_end[1] / args.col_tiles, rt_end2 = args.tile_end[2] / args.col_tiles;

    // A workgroup keeps one column tile and walks row tiles, their chunks as one sequence of steps; the loads of a step
    // are issued during the products of the step before, also across the end of a tile, so that only the very first
    // chunk is waited for.  Which tiles: workgroups are dealt to the eight XCDs in turn (workgroup w runs on XCD
    // w % 8), and each XCD has an L2 of its own.  The column tiles of one row tile share its rows, so they go to
    // workgroups of the same XCD that start together and do the same amount of work: w = 8 q + x takes column tile
    // q % col_tiles of the row tiles x + 8 (q / col_tiles) + k * stride.  The rows then come from HBM once and from
    // L2 for the other column tiles (the first layer's data gradient has three: its fetches were three times its
    // inputs when one workgroup took the column tiles of a row tile one after the other).
    struct Cursor {
        const float* rows;          // kRank1: the per-row factors
        const float* head_w;
        const float* deriv;
        const float* wt;            // the type's weights (column tile 0)
        int row0, n, t;
        int rt, ctile, chunk;
        bool live;
    };
    auto open_row_tile = [&](Cursor& c) {
        c.live = c.rt < row_tiles;
        if (!c.live) return;
        const int t = (c.rt >= rt_end0) + (c.rt >= rt_end1) + (c.rt >= rt_end2);
        const int first = t == 0 ? 0 : t == 1 ? rt_end0 : t == 2 ? rt_end1 : rt_end2;
        c.t = t;
        c.rows = kRank1 ? args.scale[t] : args.rows[t];
        c.head_w = args.head_w[t];
        c.deriv = args.deriv[t];
        c.wt = args.wt[t];
        c.row0 = (c.rt - first) * kTileRows;
        c.n = args.n[t];
        c.chunk = 0;
    };
    const int wg_x = static_cast<int>(blockIdx.x) & 7, wg_q = static_cast<int>(blockIdx.x) >> 3;
    const int rt_stride = (static_cast<int>(gridDim.x) >> 3) / col_tiles * 8;       // the grid is a multiple of 8 col_tiles
    auto advance = [&](Cursor& c) {
        if (++c.chunk < chunks) return;
        c.rt += rt_stride;
        open_row_tile(c);
    };

    v4 ra[kAPieces], rb[kCT][kBPieces];
    auto fetch = [&](const Cursor& c) {
#pragma unroll
        for (int u = 0; u < kAPieces; ++u) {
            const int p = tid + kThreads * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            const int gr = min(c.row0 + r, c.n - 1);            // past the end: the last row again, never stored
            const size_t at = static_cast<size_t>(gr) * K + c.chunk * kChunk + k4;
            if constexpr (kRank1) ra[u] = rank1_piece(c.rows, c.head_w, gr, c.chunk * kChunk + k4);
            else ra[u] = *reinterpret_cast<const v4*>(c.rows + at);
            if constexpr (kDeriv) {
                const v4 h = *reinterpret_cast<const v4*>(c.deriv + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) ra[u][e] *= h[e] >= 0.f ? 1.0f : fmaf(h[e], inv_alpha, 1.0f);
            }
        }
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
            const float* wt = c.wt + static_cast<size_t>(c.ctile * kCT + ct) * kTileCols * K;
#pragma unroll
            for (int u = 0; u < kBPieces; ++u) {
                const int p = tid + kThreads * u;
                const int r = p >> 3, k4 = (p & 7) << 2;
                rb[ct][u] = *reinterpret_cast<const v4*>(wt + static_cast<size_t>(r) * K + c.chunk * kChunk + k4);
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int u = 0; u < kAPieces; ++u) {
            const int p = tid + kThreads * u;
            const int r = p >> 3, k4 = (p & 7) << 2;
            unsigned lo[3], hi[3];
            split_pair(ra[u][0], ra[u][1], lo[0], lo[1], lo[2]);
            split_pair(ra[u][2], ra[u][3], hi[0], hi[1], hi[2]);
#pragma unroll
            for (int q = 0; q < 3; ++q) *reinterpret_cast<u2v*>(&S.a[q][r][k4]) = u2v{lo[q], hi[q]};
        }
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct) {
#pragma unroll
            for (int u = 0; u < kBPieces; ++u) {
                const int p = tid + kThreads * u;
                const int r = p >> 3, k4 = (p & 7) << 2;
                unsigned lo[3], hi[3];
                split_pair(rb[ct][u][0], rb[ct][u][1], lo[0], lo[1], lo[2]);
                split_pair(rb[ct][u][2], rb[ct][u][3], hi[0], hi[1], hi[2]);
#pragma unroll
                for (int q = 0; q < 3; ++q) *reinterpret_cast<u2v*>(&S.b[ct][q][r][k4]) = u2v{lo[q], hi[q]};
            }
        }
    };

    // this wavefront's part: rows wr*32.., columns wc*64.. (two 32 x 32 blocks across)
    const int wr = kTileCols == 128 ? (wave >> 1) : wave, wc = kTileCols == 128 ? (wave & 1) : 0;
    const int l32 = lane & 31, half = lane >> 5;
    v16 acc[kCT][1][2];
    auto clear = [&]() {
#pragma unroll
        for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[ct][0][j][e] = 0.f;
    };
    clear();

    Cursor load;                 // the step whose loads are in registers
    load.rt = wg_x + 8 * (wg_q / col_tiles);
    load.ctile = wg_q % col_tiles;
    open_row_tile(load);
    if (!load.live) return;
    fetch(load);
    for (;;) {
        // the tile that the staged chunk belongs to (for its epilogue)
        const int t = load.t, row0 = load.row0, n = load.n, ctile = load.ctile;
        const bool last_chunk = load.chunk == chunks - 1;
        stage();                                     // the chunk fetched during the previous products
        __syncthreads();
        advance(load);
        if (load.live) fetch(load);                  // in flight while this chunk is multiplied
#pragma unroll
        for (int q = 0; q < kChunk / 16; ++q) {
            // eight consecutive k of this lane's row / column: k = 16 q + 8 half + (0..7)
            bf16x8 av[3];
#pragma unroll
            for (int m = 0; m < 3; ++m)
                av[m] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u4v*>(&S.a[m][wr * 32 + l32][q * 16 + half * 8]));
#pragma unroll
            for (int ct = 0; ct < kCT; ++ct) {
                bf16x8 bv[2][3];
#pragma unroll
                for (int m = 0; m < 3; ++m)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        bv[j][m] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u4v*>(&S.b[ct][m][wc * 64 + j * 32 + l32][q * 16 + half * 8]));
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    // smallest partial products first
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[2], bv[j][0], acc[ct][0][j], 0, 0, 0);
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][2], acc[ct][0][j], 0, 0, 0);
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[j][1], acc[ct][0][j], 0, 0, 0);
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1], bv[j][0], acc[ct][0][j], 0, 0, 0);
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][1], acc[ct][0][j], 0, 0, 0);
                    acc[ct][0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[0], bv[j][0], acc[ct][0][j], 0, 0, 0);
                }
            }
        }
        __syncthreads();                             // everyone has read the chunk before it is overwritten
        if (last_chunk) {
#pragma unroll
            for (int ct = 0; ct < kCT; ++ct) {
                const int col0 = (ctile * kCT + ct) * kTileCols;
                const float* __restrict__ bias = args.bias[t];
                float bj[2], hw[2] = {0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    bj[j] = bias ? bias[col0 + wc * 64 + j * 32 + l32] : 0.f;
                    if constexpr (kHead) hw[j] = args.head_w[t][col0 + j * 32 + l32];
                }
                tile_epilogue<kCelu, kHead, 1>(acc[ct], bj, hw, args.head_b[t], args.out[t], args.head_out[t], n, args.n_out,
                                               row0 + wr * 32, col0 + wc * 64, l32, half, alpha, inv_alpha);
            }
            clear();
            if (!load.live) break;
        }
    }
}

// compute units of the current device (looked up once per device)
int compute_units()
{
    static int cached[64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    int cus = __atomic_load_n(&cached[device], __ATOMIC_RELAXED);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
        __atomic_store_n(&cached[device], cus, __ATOMIC_RELAXED);
    }
    return cus;
}

enum class Extra { kNone, kHead, kRank1 };

// The products run on the bfloat16 matrix instructions with three-way split operands (dense_split_kernel) unless
// KHAN_DENSE_MATRIX=f32 (read once) asks for the float32 matrix instructions.
bool split_products()
{
    static const bool on = [] {
        const char* v = std::getenv("KHAN_DENSE_MATRIX");
        return !(v != nullptr && std::strcmp(v, "f32") == 0);
    }();
    return on;
}

template <int kTileCols, int kK>
hipError_t launch_tiles_k(const DenseArgs& a, int run, bool celu, bool deriv, Extra extra, float alpha, hipStream_t stream)
{
    const float inv_alpha = 1.0f / alpha;
    if (split_products()) {
        if constexpr (kTileCols == 128) {
            if (a.col_tiles == 3 && extra == Extra::kNone) {
                // the three column tiles of a 384-wide output at once: one workgroup per CU
                const int row_tiles = run / a.col_tiles;
                int groups = compute_units() / 8;
                const int needed = (row_tiles + 7) / 8;
                if (groups > needed) groups = needed;
                if (groups < 1) groups = 1;
                const dim3 grid(static_cast<unsigned>(groups * 8)), block(512);
                if (celu && !deriv) dense_split_kernel<128, true, false, false, false, 3><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
                else if (!celu && !deriv) dense_split_kernel<128, false, false, false, false, 3><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
                else if (!celu && deriv) dense_split_kernel<128, false, true, false, false, 3><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
                else dense_split_kernel<128, true, true, false, false, 3><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
                return hipGetLastError();
            }
        }
        constexpr int kThreads = kTileCols * 4;
        // as many workgroups as stay resident (61 / 46 KB of LDS: two / three per CU), each walking row tiles
        // (the grid is a multiple of 8 x column tiles: see the kernel)
        const int row_tiles = run / a.col_tiles;
        const int resident = compute_units() * (kTileCols == 128 ? 2 : 3);
        const int unit = 8 * a.col_tiles;
        int groups = resident / unit;                     // row tiles in flight per XCD
        const int needed = (row_tiles + 7) / 8;
        if (groups > needed) groups = needed;
        if (groups < 1) groups = 1;
        const dim3 grid(static_cast<unsigned>(groups * unit)), block(kThreads);
        if (extra == Extra::kRank1) dense_split_kernel<kTileCols, false, true, false, true><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
        else if (extra == Extra::kHead) {
            if constexpr (kTileCols == 64) {
                if (celu) dense_split_kernel<64, true, false, true, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
                else dense_split_kernel<64, false, false, true, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
            } else return hipErrorInvalidValue;
        }
        else if (celu && !deriv) dense_split_kernel<kTileCols, true, false, false, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
        else if (!celu && !deriv) dense_split_kernel<kTileCols, false, false, false, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
        else if (!celu && deriv) dense_split_kernel<kTileCols, false, true, false, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
        else dense_split_kernel<kTileCols, true, true, false, false><<<grid, block, 0, stream>>>(a, row_tiles, alpha, inv_alpha);
        return hipGetLastError();
    }
    // the widths of the reference's default network 384-128-128-64-1, forward and backward
    if constexpr ((kTileCols == 128 && kK > 0) || (kTileCols == 64 && kK == 128)) {
        // the pipelined kernel: as many workgroups as stay resident (two per CU at 72 KB of LDS, three at 54 KB)
        const int cus = compute_units();
        constexpr int kThreads = kTileCols == 128 ? 512 : 256;
        const int resident = cus * 2;
        const dim3 pgrid(static_cast<unsigned>(run < resident ? run : resident)), pblock(kThreads);
        if (extra == Extra::kRank1) dense_pipe_kernel<kTileCols, kThreads, kK, false, true, false, true><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
        else if (extra == Extra::kHead) {
            if constexpr (kTileCols == 64) {
                if (celu) dense_pipe_kernel<64, kThreads, kK, true, false, true, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
                else dense_pipe_kernel<64, kThreads, kK, false, false, true, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
            } else return hipErrorInvalidValue;
        }
        else if (celu && !deriv) dense_pipe_kernel<kTileCols, kThreads, kK, true, false, false, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
        else if (!celu && !deriv) dense_pipe_kernel<kTileCols, kThreads, kK, false, false, false, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
        else if (!celu && deriv) dense_pipe_kernel<kTileCols, kThreads, kK, false, true, false, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
        else dense_pipe_kernel<kTileCols, kThreads, kK, true, true, false, false><<<pgrid, pblock, 0, stream>>>(a, run, alpha, inv_alpha);
        return hipGetLastError();
    }
    const dim3 grid(static_cast<unsigned>(run)), block(256);
    if (extra == Extra::kRank1) dense_kernel<kTileCols, false, true, false, true><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
    else if (extra == Extra::kHead) {
        if constexpr (kTileCols == 64) {
            if (celu) dense_kernel<64, true, false, true, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
            else dense_kernel<64, false, false, true, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
        } else return hipErrorInvalidValue;
    }
    else if (celu && !deriv) dense_kernel<kTileCols, true, false, false, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
    else if (!celu && !deriv) dense_kernel<kTileCols, false, false, false, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
    else if (!celu && deriv) dense_kernel<kTileCols, false, true, false, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
    else dense_kernel<kTileCols, true, true, false, false><<<grid, block, 0, stream>>>(a, alpha, inv_alpha);
    return hipGetLastError();
}

template <int kTileCols>
hipError_t launch_tiles(const DenseArgs& a, int run, bool celu, bool deriv, Extra extra, float alpha, hipStream_t stream)
{
    if (a.k == 384) return launch_tiles_k<kTileCols, 384>(a, run, celu, deriv, extra, alpha, stream);
    if (a.k == 128) return launch_tiles_k<kTileCols, 128>(a, run, celu, deriv, extra, alpha, stream);
    if (a.k == 64) return launch_tiles_k<kTileCols, 64>(a, run, celu, deriv, extra, alpha, stream);
    return launch_tiles_k<kTileCols, 0>(a, run, celu, deriv, extra, alpha, stream);
}

// fills the tile bookkeeping and launches
hipError_t launch_filled(DenseArgs& a, const int32_t n[4], bool celu, bool deriv, Extra extra, float alpha, hipStream_t stream)
{
    const int tile_cols = (a.n_out % 128 == 0) ? 128 : 64;
    a.col_tiles = a.n_out / tile_cols;
    int64_t run = 0;
    for (int t = 0; t < 4; ++t) {
        a.n[t] = n[t];
        run += static_cast<int64_t>((n[t] + kTileRows - 1) / kTileRows) * a.col_tiles;
        a.tile_end[t] = static_cast<int>(run);
    }
    if (run == 0) return hipSuccess;
    if (run > INT32_MAX) return hipErrorInvalidValue;
    if (tile_cols == 128) return launch_tiles<128>(a, static_cast<int>(run), celu, deriv, extra, alpha, stream);
    return launch_tiles<64>(a, static_cast<int>(run), celu, deriv, extra, alpha, stream);
}

}  // namespace

// k: a multiple of 32; n_out: a multiple of 64.  bias and deriv_of may be null (as arrays, or entry by entry).
hipError_t launch_dense(const float* const rows[4], const int32_t n[4], int32_t k, int32_t n_out,
                        const float* const wt[4], const float* const bias[4], bool celu, float alpha,
                        const float* const deriv_of[4], float* const out[4], hipStream_t stream)
{
    DenseArgs a = {};
    a.k = k;
    a.n_out = n_out;
    bool deriv = false;
    for (int t = 0; t < 4; ++t) {
        a.rows[t] = rows[t];
        a.deriv[t] = deriv_of ? deriv_of[t] : nullptr;
        a.wt[t] = wt[t];
        a.bias[t] = bias ? bias[t] : nullptr;
        a.out[t] = out[t];
        if (n[t] > 0 && a.deriv[t]) deriv = true;
    }
    return launch_filled(a, n, celu, deriv, Extra::kNone, alpha, stream);
}

// The last hidden layer (n_out = 64) together with the output layer behind it:
// out[t] = act(rows[t] . W + b) as above, and head_out[t][r] = out[t][r, :] . head_w[t] + head_b[t][0].
hipError_t launch_dense_head(const float* const rows[4], const int32_t n[4], int32_t k, int32_t n_out,
                             const float* const wt[4], const float* const bias[4], bool celu, float alpha,
                             const float* const head_w[4], const float* const head_b[4], float* const out[4],
                             float* const head_out[4], hipStream_t stream)
{
    if (n_out != 64) return hipErrorInvalidValue;
    DenseArgs a = {};
    a.k = k;
    a.n_out = n_out;
    for (int t = 0; t < 4; ++t) {
        a.rows[t] = rows[t];
        a.wt[t] = wt[t];
        a.bias[t] = bias ? bias[t] : nullptr;
        a.out[t] = out[t];
        a.head_w[t] = head_w[t];
        a.head_b[t] = head_b ? head_b[t] : nullptr;
        a.head_out[t] = head_out[t];
    }
    return launch_filled(a, n, celu, false, Extra::kHead, alpha, stream);
}

// The way back through the output layer and the last hidden layer (weights W [n_out, k] as stored, CELU outputs h):
// out[t] = (scale[t][r] * head_w[t][c] * CELU'(h[t][r, c])) . W^T-as-stored, i.e. the gradient with respect to the
// last hidden layer's input, given the gradient `scale` with respect to each row's output value.
hipError_t launch_dense_head_grad(const float* const scale[4], const float* const head_w[4], const int32_t n[4], int32_t k,
                                  int32_t n_out, const float* const wt[4], float alpha, const float* const deriv_of[4],
                                  float* const out[4], hipStream_t stream)
{
    DenseArgs a = {};
    a.k = k;
    a.n_out = n_out;
    for (int t = 0; t < 4; ++t) {
        a.scale[t] = scale[t];
        a.head_w[t] = head_w[t];
        a.deriv[t] = deriv_of[t];
        a.wt[t] = wt[t];
        a.out[t] = out[t];
    }
    return launch_filled(a, n, false, true, Extra::kRank1, alpha, stream);
}

hipError_t launch_dense_first(const float* const rows[4], const int32_t n[4], const float* const wt[4],
                              const float* const bias[4], bool celu, float alpha, float* const out[4],
                              hipStream_t stream)
{
    return launch_dense(rows, n, kFeats, 128, wt, bias, celu, alpha, nullptr, out, stream);
}

}  // namespace khan
