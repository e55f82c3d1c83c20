// What the HDLA layer does between its projections and the attention operator, in one pass per direction:
//     q = silu(q_raw) [l2-normalised per head],  k = l2norm(silu(k_raw)),  v = silu(v_raw) [l2-normalised],
//     beta = beta_scale * sigmoid(bet_raw),        log_f = logsigmoid(f)
// (HRDPLR/hdla_custom.py:214-251: activations :228-230, head split :233-236, l2_norm :247-251 with
// HRDPLR/normalizations/l2_norm.py:4-14, beta :221-224, log decay :219).  The reference runs one elementwise kernel
// per step of that list and autograd one more each on the way back; here q_raw, k_raw, v_raw, bet_raw are column
// ranges of one projection output y [rows, ldy] (read in place, strided), the results leave as the contiguous
// [rows, H, D] tensors the operator takes, and the backward pass writes the gradient of y's column ranges in place.
//
// HBM-bound byte work: a (row, head) pair is D elements = LPR lanes of 16 bytes, 64/LPR pairs per wavefront pass, the
// sums over a head are butterflies inside the wavefront.
#include "hdla_common.cuh"
#include "../../include/hdla_hip.h"

namespace hdla {

struct PreArgs {
    const void* y;                            // [rows, ldy]
    void *q, *k, *v, *beta;                   // forward outputs: [rows, H, D] x 3, [rows, H]
    const void *dq, *dk, *dv, *dbeta;         // backward inputs
    void* dy;                                 // backward output [rows, ldy]: the four column ranges are written
    long long nslot, nsg;                     // rows * H, wavefront passes
    int H, D, ldy, cq, ck, cv, cb;            // column offsets in y; cb < 0: no beta
    int lpr_log2, norm_q, norm_k, norm_v;
    float beta_scale, eps_d;                  // eps_d = D * eps: o = u / sqrt(sum u^2 + D eps)
};

typedef unsigned pre_u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct PrePiece;
template <> struct PrePiece<bf16> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void ld(const void* base, long long elem, float (&f)[8]) {
        const pre_u32x4 r = *reinterpret_cast<const pre_u32x4*>(static_cast<const bf16*>(base) + elem);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(r[i] << 16);
            f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void st(void* base, long long elem, const float (&f)[8]) {
        pre_u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = (uint32_t)f2bf(f[2 * i]) | ((uint32_t)f2bf(f[2 * i + 1]) << 16);
        *reinterpret_cast<pre_u32x4*>(static_cast<bf16*>(base) + elem) = r;
    }
};
template <> struct PrePiece<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void ld(const void* base, long long elem, float (&f)[4]) {
        const f32x4 r = *reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem);
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = r[i];
    }
    static __device__ __forceinline__ void st(void* base, long long elem, const float (&f)[4]) {
        f32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = f[i];
        *reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem) = r;
    }
};

template <typename T> __device__ __forceinline__ float pre_sigmoid(float x) { return 1.f / (1.f + exp_t<T>(-x)); }

// u = silu(x) in place; returns nothing.  sg[j] keeps sigmoid(x) for the backward pass.
template <typename T, int N> __device__ __forceinline__ void silu_fwd(float (&x)[N], float (&sg)[N]) {
#pragma unroll
    for (int j = 0; j < N; ++j) { sg[j] = pre_sigmoid<T>(x[j]); x[j] *= sg[j]; }
}

template <typename T>
__global__ __launch_bounds__(256) void layer_pre_fwd_kernel(PreArgs p) {
    constexpr int N = PrePiece<T>::N;
    const int lane = threadIdx.x & 63, lpr = 1 << p.lpr_log2, rpw = 64 >> p.lpr_log2;
    const int sl = lane & (lpr - 1), rw = lane >> p.lpr_log2;
    const long long nwave = (long long)gridDim.x * 4, wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    for (long long sg_ = wave; sg_ < p.nsg; sg_ += nwave) {
        const long long slot = sg_ * rpw + rw;
        const bool live = slot < p.nslot;
        const long long row = live ? slot / p.H : 0;
        const int h = live ? (int)(slot - row * p.H) : 0;
        const long long in = row * p.ldy + (long long)h * p.D + sl * N, out = slot * p.D + sl * N;
        float q[N], k[N], v[N], s[N];
        if (live) {
            PrePiece<T>::ld(p.y, in + p.cq, q);
            PrePiece<T>::ld(p.y, in + p.ck, k);
            PrePiece<T>::ld(p.y, in + p.cv, v);
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) q[j] = k[j] = v[j] = 0.f;
        }
        silu_fwd<T, N>(q, s);
        silu_fwd<T, N>(k, s);
        silu_fwd<T, N>(v, s);
        float sq = 0.f, sk = 0.f, sv = 0.f;
#pragma unroll
        for (int j = 0; j < N; ++j) { sq += q[j] * q[j]; sk += k[j] * k[j]; sv += v[j] * v[j]; }
        for (int o = 1; o < lpr; o <<= 1) { sq += __shfl_xor(sq, o); sk += __shfl_xor(sk, o); sv += __shfl_xor(sv, o); }
        const float iq = p.norm_q ? 1.f / sqrtf(sq + p.eps_d) : 1.f;
        const float ik = p.norm_k ? 1.f / sqrtf(sk + p.eps_d) : 1.f;
        const float iv = p.norm_v ? 1.f / sqrtf(sv + p.eps_d) : 1.f;
#pragma unroll
        for (int j = 0; j < N; ++j) { q[j] *= iq; k[j] *= ik; v[j] *= iv; }
        if (live) {
            PrePiece<T>::st(p.q, out, q);
            PrePiece<T>::st(p.k, out, k);
            PrePiece<T>::st(p.v, out, v);
            if (p.cb >= 0 && sl == 0) {
                const float b = ld_elem(static_cast<const T*>(p.y) + row * p.ldy + p.cb + h);
                st_elem(static_cast<T*>(p.beta) + slot, p.beta_scale * pre_sigmoid<T>(b));
            }
        }
    }
}

// one of q, k, v on the way back: x raw input (in), g gradient of the output (in) -> gradient of the raw input (in g)
template <typename T, int N>
__device__ __forceinline__ void pre_bwd_one(float (&x)[N], float (&g)[N], bool norm, float eps_d, int lpr) {
    float s[N], u[N];
#pragma unroll
    for (int j = 0; j < N; ++j) { u[j] = x[j]; }
    silu_fwd<T, N>(u, s);
    if (norm) {          // uniform over the launch
        float su = 0.f, sd = 0.f;
#pragma unroll
        for (int j = 0; j < N; ++j) { su += u[j] * u[j]; sd += u[j] * g[j]; }
        for (int o = 1; o < lpr; o <<= 1) { su += __shfl_xor(su, o); sd += __shfl_xor(sd, o); }
        const float inv = 1.f / sqrtf(su + eps_d);
        const float proj = sd * inv * inv;                 // sum(o * do) / |.|: with o = u inv, du = inv (do - o sum(o do))
#pragma unroll
        for (int j = 0; j < N; ++j) g[j] = inv * (g[j] - u[j] * proj);
    }
#pragma unroll
    for (int j = 0; j < N; ++j) g[j] *= s[j] * (1.f + x[j] * (1.f - s[j]));       // silu'(x)
}

template <typename T>
__global__ __launch_bounds__(256) void layer_pre_bwd_kernel(PreArgs p) {
    constexpr int N = PrePiece<T>::N;
    const int lane = threadIdx.x & 63, lpr = 1 << p.lpr_log2, rpw = 64 >> p.lpr_log2;
    const int sl = lane & (lpr - 1), rw = lane >> p.lpr_log2;
    const long long nwave = (long long)gridDim.x * 4, wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    for (long long sg_ = wave; sg_ < p.nsg; sg_ += nwave) {
        const long long slot = sg_ * rpw + rw;
        const bool live = slot < p.nslot;
        const long long row = live ? slot / p.H : 0;
        const int h = live ? (int)(slot - row * p.H) : 0;
        const long long in = row * p.ldy + (long long)h * p.D + sl * N, out = slot * p.D + sl * N;
        float q[N], k[N], v[N], gq[N], gk[N], gv[N];
        if (live) {
            PrePiece<T>::ld(p.y, in + p.cq, q);
            PrePiece<T>::ld(p.y, in + p.ck, k);
            PrePiece<T>::ld(p.y, in + p.cv, v);
            PrePiece<T>::ld(p.dq, out, gq);
            PrePiece<T>::ld(p.dk, out, gk);
            PrePiece<T>::ld(p.dv, out, gv);
        } else {
#pragma unroll
            for (int j = 0; j < N; ++j) q[j] = k[j] = v[j] = gq[j] = gk[j] = gv[j] = 0.f;
        }
        pre_bwd_one<T, N>(q, gq, p.norm_q != 0, p.eps_d, lpr);
        pre_bwd_one<T, N>(k, gk, p.norm_k != 0, p.eps_d, lpr);
        pre_bwd_one<T, N>(v, gv, p.norm_v != 0, p.eps_d, lpr);
        if (live) {
            PrePiece<T>::st(p.dy, in + p.cq, gq);
            PrePiece<T>::st(p.dy, in + p.ck, gk);
            PrePiece<T>::st(p.dy, in + p.cv, gv);
            if (p.cb >= 0 && sl == 0) {
                const float b = pre_sigmoid<T>(ld_elem(static_cast<const T*>(p.y) + row * p.ldy + p.cb + h));
                const float g = ld_elem(static_cast<const T*>(p.dbeta) + slot);
                st_elem(static_cast<T*>(p.dy) + row * p.ldy + p.cb + h, g * p.beta_scale * b * (1.f - b));
            }
        }
    }
}

// log_f = logsigmoid(f) = min(f, 0) - log(1 + exp(-|f|)) and its gradient df = dlog_f * sigmoid(-f), 16 bytes a lane
template <typename T, bool BWD>
__global__ __launch_bounds__(256) void logsigmoid_kernel(const void* x, const void* dy, void* out, long long npiece) {
    constexpr int N = PrePiece<T>::N;
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < npiece; i += stride) {
        float f[N], g[N];
        PrePiece<T>::ld(x, i * N, f);
        if (BWD) PrePiece<T>::ld(dy, i * N, g);
#pragma unroll
        for (int j = 0; j < N; ++j) {
            if (BWD) f[j] = g[j] * pre_sigmoid<T>(-f[j]);
            else {
                // log(1 + e) for e = exp(-|f|) in (0, 1]: the accurate routine for fp32 results; for bf16 results the
                // hardware logarithm, with the first term of the series where 1 + e would round e away
                const float e = exp_t<T>(-fabsf(f[j]));
                const float l = sizeof(T) == 4 ? log1pf(e) : (e < 1e-4f ? e : __logf(1.f + e));
                f[j] = fminf(f[j], 0.f) - l;
            }
        }
        PrePiece<T>::st(out, i * N, f);
    }
}

static bool pre_al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static int pre_config(const hdla_pre_dims* d, PreArgs& a, unsigned& nwg) {
    if (!d) return HDLA_ERR_NULL;
    if (d->dtype != HDLA_BF16 && d->dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    const int n = d->dtype == HDLA_BF16 ? 8 : 4;
    if (d->rows < 0 || d->H <= 0 || d->D <= 0 || d->D % n || !(d->eps >= 0.f)) return HDLA_ERR_SHAPE;
    const int lpr = d->D / n;
    if (lpr > 64 || (lpr & (lpr - 1))) return HDLA_ERR_SHAPE;                 // a head: a power of two of lanes
    const long long hd = (long long)d->H * d->D;
    if (d->ldy % n || d->col_q % n || d->col_k % n || d->col_v % n) return HDLA_ERR_ALIGN;
    if (d->col_q < 0 || d->col_k < 0 || d->col_v < 0) return HDLA_ERR_SHAPE;
    const long long ends[3] = {d->col_q + hd, d->col_k + hd, d->col_v + hd};
    for (long long e : ends) if (e > d->ldy) return HDLA_ERR_SHAPE;
    if (d->col_beta >= 0 && (long long)d->col_beta + d->H > d->ldy) return HDLA_ERR_SHAPE;
    if (d->rows > (1LL << 40) / d->H) return HDLA_ERR_SHAPE;
    a = PreArgs{};
    a.nslot = d->rows * d->H; a.H = d->H; a.D = d->D; a.ldy = d->ldy;
    a.cq = d->col_q; a.ck = d->col_k; a.cv = d->col_v; a.cb = d->col_beta < 0 ? -1 : d->col_beta;
    a.lpr_log2 = 0;
    while ((1 << a.lpr_log2) < lpr) ++a.lpr_log2;
    const int rpw = 64 >> a.lpr_log2;
    a.nsg = (a.nslot + rpw - 1) / rpw;
    a.norm_q = d->norm_q != 0; a.norm_k = d->norm_k != 0; a.norm_v = d->norm_v != 0;
    a.beta_scale = d->beta_scale; a.eps_d = d->eps * (float)d->D;
    const long long per_wave = a.nsg >= 16384 ? 4 : 1;          // passes per wavefront; few when the problem is small
    long long w = (a.nsg + 4 * per_wave - 1) / (4 * per_wave);
    nwg = (unsigned)(w < 1 ? 1 : (w > 8192 ? 8192 : w));
    return HDLA_OK;
}

}  // namespace hdla

using namespace hdla;

extern "C" int hdla_layer_pre_fwd(const hdla_pre_dims* dims, const void* y, void* q, void* k, void* v, void* beta,
                                  void* stream) {
    PreArgs a; unsigned nwg;
    const int rc = pre_config(dims, a, nwg);
    if (rc) return rc;
    if (dims->rows == 0) return HDLA_OK;
    if (!y || !q || !k || !v || (a.cb >= 0 && !beta)) return HDLA_ERR_NULL;
    if (!pre_al16(y) || !pre_al16(q) || !pre_al16(k) || !pre_al16(v)) return HDLA_ERR_ALIGN;
    a.y = y; a.q = q; a.k = k; a.v = v; a.beta = beta;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (dims->dtype == HDLA_BF16) hipLaunchKernelGGL(layer_pre_fwd_kernel<bf16>, dim3(nwg), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(layer_pre_fwd_kernel<float>, dim3(nwg), dim3(256), 0, s, a);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? HDLA_OK : (int)e;
}

extern "C" int hdla_layer_pre_bwd(const hdla_pre_dims* dims, const void* y, const void* dq, const void* dk,
                                  const void* dv, const void* dbeta, void* dy, void* stream) {
    PreArgs a; unsigned nwg;
    const int rc = pre_config(dims, a, nwg);
    if (rc) return rc;
    if (dims->rows == 0) return HDLA_OK;
    if (!y || !dq || !dk || !dv || !dy || (a.cb >= 0 && !dbeta)) return HDLA_ERR_NULL;
    if (!pre_al16(y) || !pre_al16(dq) || !pre_al16(dk) || !pre_al16(dv) || !pre_al16(dy)) return HDLA_ERR_ALIGN;
    a.y = y; a.dq = dq; a.dk = dk; a.dv = dv; a.dbeta = dbeta; a.dy = dy;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (dims->dtype == HDLA_BF16) hipLaunchKernelGGL(layer_pre_bwd_kernel<bf16>, dim3(nwg), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(layer_pre_bwd_kernel<float>, dim3(nwg), dim3(256), 0, s, a);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? HDLA_OK : (int)e;
}

static int logsigmoid_launch(int dtype, long long n, const void* x, const void* dy, void* out, bool bwd, void* stream) {
    if (dtype != HDLA_BF16 && dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    const int N = dtype == HDLA_BF16 ? 8 : 4;
    if (n < 0 || n % N) return HDLA_ERR_SHAPE;
    if (n == 0) return HDLA_OK;
    if (!x || !out || (bwd && !dy)) return HDLA_ERR_NULL;
    if (!pre_al16(x) || !pre_al16(out) || !pre_al16(dy)) return HDLA_ERR_ALIGN;
    const long long np = n / N;
    long long w = (np + 1023) / 1024;
    const dim3 grid((unsigned)(w < 1 ? 1 : (w > 8192 ? 8192 : w))), block(256);
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == HDLA_BF16) {
        if (bwd) hipLaunchKernelGGL((logsigmoid_kernel<bf16, true>), grid, block, 0, s, x, dy, out, np);
        else hipLaunchKernelGGL((logsigmoid_kernel<bf16, false>), grid, block, 0, s, x, dy, out, np);
    } else {
        if (bwd) hipLaunchKernelGGL((logsigmoid_kernel<float, true>), grid, block, 0, s, x, dy, out, np);
        else hipLaunchKernelGGL((logsigmoid_kernel<float, false>), grid, block, 0, s, x, dy, out, np);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? HDLA_OK : (int)e;
}

extern "C" int hdla_logsigmoid_fwd(int dtype, int64_t n, const void* x, void* y, void* stream) {
    return logsigmoid_launch(dtype, n, x, nullptr, y, false, stream);
}

extern "C" int hdla_logsigmoid_bwd(int dtype, int64_t n, const void* x, const void* dy, void* dx, void* stream) {
    return logsigmoid_launch(dtype, n, x, dy, dx, true, stream);
}
