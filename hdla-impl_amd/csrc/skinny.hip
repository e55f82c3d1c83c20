// dW [K, N] = dY [M, K]^T * X0 [M, N] for a narrow N (64 or 128) and many rows M, bf16 in, fp32 accumulation, bf16 out.
//
// This is the weight gradient of the second half of the HDLA layer's low-rank projections (f_proj and output_gate:
// Linear(embed_dim -> head_dim) followed by Linear(head_dim -> embed_dim), HRDPLR/hdla_custom.py:117-121,151-155; in the
// reference a BLAS call inside autograd).  The output is tiny (K x N) and the contraction runs over all rows, so a
// BLAS kernel tiled over the output has 16 workgroups to work with; here the rows are split as well: a workgroup owns
// 32 columns of dY and one range of rows, its four wavefronts take every fourth 16-row tile of that range (16 bytes a
// lane from dY and from X0), add their sums through LDS, and leave a fp32 partial result; a second small kernel adds
// the partial results of the row ranges in a fixed order.
//
// The contraction index (the row) must be the inner index of both MFMA operands, and both are stored with the row
// outermost, so each 16 x 16 tile is transposed on its way in by one product with the identity (exact in bf16).
#include "hdla_common.cuh"
#include "../../include/hdla_hip.h"

namespace hdla {

// Two 16 x 16 tiles from one 16-byte load per lane: lane (g, c) reads elements 8g .. 8g+7 of row c of a 16 x 32 block;
// the first four are the fragment of tile A, the last four of tile B, where tile A holds the block's columns
// 8j + 0..3 and tile B the columns 8j + 4..7 (j = 0..3).  Element e = 0..15 of a tile's column index is therefore
// column 8 (e / 4) + e % 4 (+ 4 for tile B) of the block.
__device__ __forceinline__ void ld_two_tiles(const bf16* p, bool ok, Frag<bf16>& a, Frag<bf16>& b) {
    s16x8 x = *reinterpret_cast<const s16x8*>(p);
    const s16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    x = ok ? x : z;
    a.v = __builtin_shufflevector(x, x, 0, 1, 2, 3);
    b.v = __builtin_shufflevector(x, x, 4, 5, 6, 7);
}

template <int N>
__global__ __launch_bounds__(256) void skinny_wgrad_kernel(const bf16* __restrict__ dY, long long ldy,
                                                           const bf16* __restrict__ X0, long long ldx,
                                                           float* __restrict__ part, int M, int K, int rows_per) {
    constexpr int ZP = N / 32;                                 // 32-column blocks of X0
    __shared__ f32x4 red[3][2 * 2 * ZP][64];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
    const int k0 = blockIdx.x * 32, s = blockIdx.y;
    const long long rbeg = (long long)s * rows_per;
    const long long rend = rbeg + rows_per < M ? rbeg + rows_per : M;
    const Frag<bf16> id = ident_frag<bf16>();
    f32x4 acc[2][2 * ZP];                                      // [tile of dY's 32 columns][tile of X0's columns]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2 * ZP; ++b) acc[a][b] = zero4();
    // the four wavefronts take every fourth 16-row tile of the range
#pragma unroll 4
    for (long long r0 = rbeg + 16 * w; r0 < rend; r0 += 64) {
        const bool ok = r0 + c < rend;
        const long long row = ok ? r0 + c : rbeg;              // a readable row on every lane
        Frag<bf16> x[2], z[2 * ZP];
        ld_two_tiles(dY + row * ldy + k0 + 8 * g, ok, x[0], x[1]);
#pragma unroll
        for (int b = 0; b < ZP; ++b) ld_two_tiles(X0 + row * ldx + 32 * b + 8 * g, ok, z[2 * b], z[2 * b + 1]);
        // transposed tiles: rows = columns of the block, inner index = row of the range
        x[0] = transpose(x[0], id);
        x[1] = transpose(x[1], id);
#pragma unroll
        for (int b = 0; b < 2 * ZP; ++b) {
            const Frag<bf16> zt = transpose(z[b], id);
            acc[0][b] = mm(x[0], zt, acc[0][b]);
            acc[1][b] = mm(x[1], zt, acc[1][b]);
        }
    }
    if (w) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2 * ZP; ++b) red[w - 1][a * 2 * ZP + b][lane] = acc[a][b];
    }
    __syncthreads();
    if (w) return;
    // lane (g, c) register i of acc[a][b]: dY column k0 + 8 (c / 4) + c % 4 + 4 a,
    //                                      X0 column 32 (b / 2) + 8 g + 4 (b % 2) + i
    const int krow = k0 + 8 * (c >> 2) + (c & 3);
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2 * ZP; ++b) {
            const f32x4 v = acc[a][b] + red[0][a * 2 * ZP + b][lane] + red[1][a * 2 * ZP + b][lane] + red[2][a * 2 * ZP + b][lane];
            *reinterpret_cast<f32x4*>(part + ((long long)s * K + krow + 4 * a) * N + 32 * (b >> 1) + 8 * g + 4 * (b & 1)) = v;
        }
}

// dW = sum over the row ranges of their partial results, eight outputs a thread
__global__ __launch_bounds__(256) void skinny_wgrad_sum_kernel(const float* __restrict__ part, bf16* __restrict__ dW,
                                                               long long kn, int S) {
    const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= kn) return;
    f32x4 a = zero4(), b = zero4();
    for (int s = 0; s < S; ++s) {
        a += *reinterpret_cast<const f32x4*>(part + s * kn + i);
        b += *reinterpret_cast<const f32x4*>(part + s * kn + i + 4);
    }
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 o;
    o[0] = (uint32_t)f2bf(a[0]) | ((uint32_t)f2bf(a[1]) << 16);
    o[1] = (uint32_t)f2bf(a[2]) | ((uint32_t)f2bf(a[3]) << 16);
    o[2] = (uint32_t)f2bf(b[0]) | ((uint32_t)f2bf(b[1]) << 16);
    o[3] = (uint32_t)f2bf(b[2]) | ((uint32_t)f2bf(b[3]) << 16);
    *reinterpret_cast<u32x4*>(dW + i) = o;
}

// row ranges: enough workgroups for the chip (and, when there are many rows, several per CU, about 1024 rows each, so
// that enough loads are in flight to cover the latency of HBM), whole 16-row tiles each
static int wgrad_split(long long M, int K, int& rows_per) {
    const int kb = K / 32;
    long long S = (256 + kb - 1) / kb;
    const long long by_rows = M / 1024, most = (2048 + kb - 1) / kb;
    if (by_rows > S) S = by_rows < most ? by_rows : most;
    const long long tiles = (M + 15) / 16;
    if (S > tiles) S = tiles;
    if (S < 1) S = 1;
    rows_per = (int)(((tiles + S - 1) / S) * 16);
    return (int)((M + rows_per - 1) / rows_per);
}

}  // namespace hdla

using namespace hdla;

static int wgrad_check(int dtype, int64_t M, int32_t N, int32_t K) {
    if (dtype != HDLA_BF16) return HDLA_ERR_DTYPE;
    if (M <= 0 || M > 0x7fffffffLL || (N != 64 && N != 128) || K <= 0 || K % 64) return HDLA_ERR_SHAPE;
    return HDLA_OK;
}

extern "C" size_t hdla_skinny_wgrad_workspace_bytes(int dtype, int64_t M, int32_t N, int32_t K) {
    if (wgrad_check(dtype, M, N, K)) return 0;
    int rows_per;
    const int S = wgrad_split(M, K, rows_per);
    return (size_t)S * K * N * sizeof(float);
}

extern "C" int hdla_skinny_wgrad(int dtype, int64_t M, int32_t N, int32_t K, const void* dY, int64_t ldy,
                                 const void* X0, int64_t ldx, void* dW, void* workspace, size_t workspace_bytes,
                                 void* stream) {
    const int rc = wgrad_check(dtype, M, N, K);
    if (rc) return rc;
    if (ldy < K || ldx < N) return HDLA_ERR_SHAPE;
    if (!dY || !X0 || !dW) return HDLA_ERR_NULL;
    const auto al = [](const void* p, int a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    if (!al(dY, 16) || !al(X0, 16) || !al(dW, 16) || ldy % 8 || ldx % 8) return HDLA_ERR_ALIGN;
    int rows_per;
    const int S = wgrad_split(M, K, rows_per);
    const size_t need = (size_t)S * K * N * sizeof(float);
    if (!workspace || !al(workspace, 16) || workspace_bytes < need) return HDLA_ERR_WORKSPACE;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(K / 32, S), block(256);
    float* part = static_cast<float*>(workspace);
    const bf16* a = static_cast<const bf16*>(dY);
    const bf16* b = static_cast<const bf16*>(X0);
    if (N == 64) hipLaunchKernelGGL((skinny_wgrad_kernel<64>), grid, block, 0, s, a, (long long)ldy, b, (long long)ldx, part, (int)M, (int)K, rows_per);
    else hipLaunchKernelGGL((skinny_wgrad_kernel<128>), grid, block, 0, s, a, (long long)ldy, b, (long long)ldx, part, (int)M, (int)K, rows_per);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    const long long kn = (long long)K * N;
    hipLaunchKernelGGL(skinny_wgrad_sum_kernel, dim3((unsigned)((kn / 8 + 255) / 256)), block, 0, s, part, static_cast<bf16*>(dW), kn, S);
    e = hipGetLastError();
    return e == hipSuccess ? HDLA_OK : (int)e;
}
