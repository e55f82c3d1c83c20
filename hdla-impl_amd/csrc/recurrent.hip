// Fused token-serial recurrent kernel (decode step and short prefills).
//
// Replaces HRDPLR/recurrent.py:26-119.  Per token
//     S <- Diag(exp(g)) S + sum_r b_r (a_r^T S) + k v^T ,   o = scale * S^T q
// with both rank terms reading the state before the decay (recurrent.py:93-100) and the output reading the
// updated state (recurrent.py:104).  For a decode step the kernel is a pure stream of the fp32 state through
// HBM (read K*V*4 bytes, write K*V*4 bytes per head), so the layout is chosen for that: one 256-thread
// workgroup owns a K x 64 column block of one head's state, every lane moves 16-byte pieces of whole 256-byte
// row segments, and all of a block's loads are in flight before the first use.  The two reductions over K
// (a^T S and q^T S) run as in-lane partial sums, two cross-lane butterfly steps and one LDS exchange between
// the four wavefronts.
//
// HD mode (p.beta given) forms the rank terms of the HDLA layer per token from (beta, k, gk) instead of reading
// them (HRDPLR/hdla_custom.py:19-43): with f = exp(gk) and s = sum_c k_c^2 f_c,
//     a_1 = -beta k,  a_2 = beta k (beta s - f),  b_1 = f k,  b_2 = k,
// each rounded to the input type as the stored tensors would be.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

__device__ __forceinline__ float ld_as_float(const bf16* p) { return bf2f(p->x); }
__device__ __forceinline__ float ld_as_float(const float* p) { return *p; }
__device__ __forceinline__ float round_as(const bf16*, float x) { return bf2f(f2bf(x)); }
__device__ __forceinline__ float round_as(const float*, float x) { return x; }
__device__ __forceinline__ float ld_gk1(const void* base, int64_t off, int is_f32) {
    return is_f32 ? reinterpret_cast<const float*>(base)[off] : bf2f(reinterpret_cast<const bf16*>(base)[off].x);
}

template <typename T, int K, int V, int BV, bool HD>
__global__ __launch_bounds__(256) void recurrent_kernel(RecurrentArgs<T> p) {
    constexpr int CG = BV / 4;        // lanes across a row segment (float4 each)
    constexpr int RG = 256 / CG;      // row groups
    constexpr int RPT = K / RG;       // state rows per thread
    static_assert(K % RG == 0 && RPT >= 1, "tile shape");
    static_assert(K <= 256, "one channel per thread in the per-token fill");
    __shared__ float sq[K], sk[K], seg[K], sa[2][K], sb[2][K], sv[BV];
    __shared__ float red[4][3][BV];

    const int nh = blockIdx.x, vb = blockIdx.y;
    const int n = nh / p.H, h = nh - n * p.H;
    const int H = p.H;
    const int tid = threadIdx.x, cg = tid % CG, rg = tid / CG, wave = tid >> 6, lane = tid & 63;
    int64_t bos, eos;
    if (p.cu) packed_bounds(p.cu, n, p.T_, bos, eos);
    else { bos = (int64_t)n * p.T_; eos = bos + p.T_; }
    const int len = (int)(eos - bos);

    const int64_t sbase = (int64_t)nh * K * V + vb * BV + 4 * cg;
    f32x4 S[RPT];
#pragma unroll
    for (int j = 0; j < RPT; ++j)
        S[j] = p.h0 ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.h0 + sbase + (int64_t)(rg + RG * j) * V)) : zero4();

    for (int step = 0; step < len; ++step) {
        const int64_t t = p.reverse ? (eos - 1 - step) : (bos + step);
        __syncthreads();
        if constexpr (HD) {
            const int64_t off = (t * H + h) * K + tid;
            float kk = 0.f, f = 0.f;
            if (tid < K) {
                kk = ld_as_float(p.k + off);
                f = exp_t<T>(ld_gk1(p.gk, off, p.gk_f32));
                sq[tid] = ld_as_float(p.q + off) * p.scale;
            }
            float part = kk * kk * f;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) part += __shfl_xor(part, o);
            if (lane == 0) red[wave][0][0] = part;
            __syncthreads();
            if (tid < K) {
                const float s = red[0][0][0] + red[1][0][0] + red[2][0][0] + red[3][0][0];
                const float beta = ld_as_float(p.beta + t * H + h);
                sk[tid] = kk;
                seg[tid] = f;
                sa[0][tid] = round_as(p.k, -beta * kk);
                sa[1][tid] = round_as(p.k, (beta * s - f) * beta * kk);
                sb[0][tid] = round_as(p.k, f * kk);
                sb[1][tid] = kk;
            }
        } else {
            for (int idx = tid; idx < K; idx += 256) {
                const int64_t off = (t * H + h) * K + idx;
                const int64_t off0 = ((t * RANK + 0) * H + h) * K + idx, off1 = ((t * RANK + 1) * H + h) * K + idx;
                sq[idx] = ld_as_float(p.q + off) * p.scale;
                sk[idx] = ld_as_float(p.k + off);
                seg[idx] = exp_t<T>(ld_gk1(p.gk, off, p.gk_f32));
                sa[0][idx] = ld_as_float(p.a + off0);
                sa[1][idx] = ld_as_float(p.a + off1);
                sb[0][idx] = ld_as_float(p.b + off0);
                sb[1][idx] = ld_as_float(p.b + off1);
            }
        }
        if (tid < BV) sv[tid] = ld_as_float(p.v + (t * H + h) * V + vb * BV + tid);
        __syncthreads();

        // a_r^T S over the block's rows
        f32x4 p0 = zero4(), p1 = zero4();
#pragma unroll
        for (int j = 0; j < RPT; ++j) {
            const int row = rg + RG * j;
            p0 += S[j] * sa[0][row];
            p1 += S[j] * sa[1][row];
        }
#pragma unroll
        for (int off = CG; off < 64; off <<= 1) {
#pragma unroll
            for (int x = 0; x < 4; ++x) { p0[x] += __shfl_xor(p0[x], off); p1[x] += __shfl_xor(p1[x], off); }
        }
        if (lane < CG) {
            *reinterpret_cast<f32x4*>(&red[wave][0][4 * cg]) = p0;
            *reinterpret_cast<f32x4*>(&red[wave][1][4 * cg]) = p1;
        }
        __syncthreads();
        f32x4 u0 = zero4(), u1 = zero4();
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            u0 += *reinterpret_cast<const f32x4*>(&red[w][0][4 * cg]);
            u1 += *reinterpret_cast<const f32x4*>(&red[w][1][4 * cg]);
        }
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(&sv[4 * cg]);
        f32x4 po = zero4();
#pragma unroll
        for (int j = 0; j < RPT; ++j) {
            const int row = rg + RG * j;
            S[j] = S[j] * seg[row] + u0 * sb[0][row] + u1 * sb[1][row] + v4 * sk[row];
            po += S[j] * sq[row];
        }
#pragma unroll
        for (int off = CG; off < 64; off <<= 1) {
#pragma unroll
            for (int x = 0; x < 4; ++x) po[x] += __shfl_xor(po[x], off);
        }
        if (lane < CG) *reinterpret_cast<f32x4*>(&red[wave][2][4 * cg]) = po;
        __syncthreads();
        if (tid < BV) {
            const float o = red[0][2][tid] + red[1][2][tid] + red[2][2][tid] + red[3][2][tid];
            st_elem(p.o + (t * H + h) * V + vb * BV + tid, o);
        }
    }
    if (p.ht) {
#pragma unroll
        for (int j = 0; j < RPT; ++j)
            __builtin_nontemporal_store(S[j], reinterpret_cast<f32x4*>(p.ht + sbase + (int64_t)(rg + RG * j) * V));
    }
}

template <typename T, int K, int V>
static hipError_t launch_recurrent_kv(const RecurrentArgs<T>& a, hipStream_t stream) {
    constexpr int BV = 64;
    dim3 grid(a.N * a.H, V / BV), block(256);
    if (a.beta) hipLaunchKernelGGL((recurrent_kernel<T, K, V, BV, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((recurrent_kernel<T, K, V, BV, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_recurrent(const RecurrentArgs<T>& a, int K, int V, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_recurrent_kv<T, 64, 64>(a, stream);
    if (K == 128 && V == 128) return launch_recurrent_kv<T, 128, 128>(a, stream);
    if (K == 64 && V == 128) return launch_recurrent_kv<T, 64, 128>(a, stream);
    if (K == 128 && V == 64) return launch_recurrent_kv<T, 128, 64>(a, stream);
    // head sizes up to 256 (the reference's token-serial kernel takes any K, HRDPLR/recurrent.py:155-176): the state
    // block of a workgroup is K x 64 values in registers, 64 per lane at K = 256
    if (K == 256 && V == 256) return launch_recurrent_kv<T, 256, 256>(a, stream);
    if (K == 256 && V == 128) return launch_recurrent_kv<T, 256, 128>(a, stream);
    if (K == 128 && V == 256) return launch_recurrent_kv<T, 128, 256>(a, stream);
    if (K == 256 && V == 64) return launch_recurrent_kv<T, 256, 64>(a, stream);
    if (K == 64 && V == 256) return launch_recurrent_kv<T, 64, 256>(a, stream);
    return hipErrorInvalidValue;
}
template hipError_t launch_recurrent<bf16>(const RecurrentArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_recurrent<float>(const RecurrentArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
