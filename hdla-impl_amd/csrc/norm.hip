// Fused normalisation with an optional gate: the operator the HDLA layer applies right after the attention
// operator (gated RMSNorm, HRDPLR/hdla_custom.py:341-345) and to q, k, v right before it (l2_norm, :247-251).
//
// Replaces _normalize_fwd / _normalize_bwd, HRDPLR/normalizations/normalize/normalize/normalize_triton.py:21-253,
// for use_mean = False and no bias or residual.  Per (row, group) of E channels:
//     x' = x * sigmoid(gate)                      gate before the norm            (normalize_triton.py:84-89)
//     sigma = sqrt(sum x'^2 / E + eps)                                            (:103)
//     o = (c / sqrt(E)) * x' / sigma * weight  [ * sigmoid(gate), gate after ]    (:104-117)
// and the matching backward pass (:186-251), with sigma recomputed instead of stored.
//
// Both passes are streams through HBM (forward: read x, gate, write o; backward: read x, gate, do, write dx, dgate),
// so the layout is chosen for that: a row (or, for short groups, 64/LPR consecutive groups) per wavefront pass, 16
// bytes per lane and piece, LPR = a power of two lanes across one group, all pieces of a pass in flight before the
// first use, sums over a group as butterflies inside the wavefront (no LDS, no barrier).  Wavefronts stride over the
// groups such that a lane always meets the same weight columns: weights are loaded once, and the weight gradient
// accumulates in registers and leaves as one partial row per (wavefront, group position), summed by a second small
// kernel in a fixed order (results do not depend on timing).
#include "hdla_common.cuh"
#include "../../include/hdla_hip.h"

namespace hdla {

struct NormArgs {
    const void *x, *gate, *weight, *d_o;
    void *o, *dx, *dgate;
    float* partial;            // [(workgroups or waves) * groups per pass][E], backward with a weight
    long long nslot;           // rows * G: groups to normalise, E consecutive elements each
    long long nsg;             // wavefront passes: ceil(nslot / (64 >> lpr_log2))
    int G, E, lpr_log2, w_f32, gate_pos;
    int wg_reduce;             // the four wavefronts of a workgroup meet the same weight columns: one partial row set
    int wg_row;                // long groups: the four wavefronts of a workgroup share one group, 256 lanes across it
    float cn, inv_e, eps;      // c / sqrt(E), 1 / E
};

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// 16 bytes of a row as floats
template <typename T> struct Piece;
template <> struct Piece<bf16> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void ld(const void* base, long long elem, float (&f)[8]) {
        const u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(static_cast<const bf16*>(base) + elem));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(r[i] << 16);
            f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void st(void* base, long long elem, const float (&f)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = (uint32_t)f2bf(f[2 * i]) | ((uint32_t)f2bf(f[2 * i + 1]) << 16);
        __builtin_nontemporal_store(r, reinterpret_cast<u32x4*>(static_cast<bf16*>(base) + elem));
    }
};
template <> struct Piece<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void ld(const void* base, long long elem, float (&f)[4]) {
        const f32x4 r = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(static_cast<const float*>(base) + elem));
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = r[i];
    }
    static __device__ __forceinline__ void st(void* base, long long elem, const float (&f)[4]) {
        f32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = f[i];
        __builtin_nontemporal_store(r, reinterpret_cast<f32x4*>(static_cast<float*>(base) + elem));
    }
};

template <int N> __device__ __forceinline__ void ld_weight(const void* w, int w_f32, int col, float (&f)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i)
        f[i] = w_f32 ? static_cast<const float*>(w)[col + i] : bf2f(static_cast<const bf16*>(w)[col + i].x);
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + __expf(-x)); }

// Where a lane stands: lane sl of the LPR lanes across one group, group position rw of the 64/LPR groups of a pass;
// `wave` counts passes' owners (wavefronts, or workgroups when a workgroup shares one long group).
struct NormLane {
    int lpr, rpw, sl, rw, wg_row;
    long long wave, nwave;
    __device__ __forceinline__ explicit NormLane(const NormArgs& p) {
        const int lane = threadIdx.x & 63;
        wg_row = p.wg_row;
        if (wg_row) {
            lpr = 256; rpw = 1; sl = threadIdx.x; rw = 0;
            nwave = gridDim.x;
            wave = blockIdx.x;
        } else {
            lpr = 1 << p.lpr_log2;
            rpw = 64 >> p.lpr_log2;
            sl = lane & (lpr - 1);
            rw = lane >> p.lpr_log2;
            nwave = (long long)gridDim.x * 4;
            wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
        }
    }
};

// Sums of a and b over the lanes of one group, on all of them.  Across the wavefronts of a workgroup the partial
// sums go through `sred` ([2][4][2] floats, alternating halves, so one barrier per call is enough); every thread of
// the workgroup makes the same calls.
__device__ __forceinline__ void group_sum(const NormLane& L, float& a, float& b, float* sred, int& buf) {
    const int width = L.wg_row ? 64 : L.lpr;
    for (int o = 1; o < width; o <<= 1) { a += __shfl_xor(a, o); b += __shfl_xor(b, o); }
    if (L.wg_row) {
        float* s = sred + buf * 8;
        if ((threadIdx.x & 63) == 0) { s[2 * (threadIdx.x >> 6)] = a; s[2 * (threadIdx.x >> 6) + 1] = b; }
        __syncthreads();
        a = (s[0] + s[2]) + (s[4] + s[6]);
        b = (s[1] + s[3]) + (s[5] + s[7]);
        buf ^= 1;
    }
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void normalize_fwd_kernel(NormArgs p) {
    constexpr int N = Piece<T>::N;
    const NormLane L(p);
    __shared__ float sred[16];
    int buf = 0;
    const bool pre = p.gate_pos == 1, post = p.gate_pos == 2;
    const int E = p.E;
    // the launch makes nwave * rpw a multiple of G: the group index of a lane's slots never changes
    const int g = (int)((L.wave * L.rpw + L.rw) % p.G);
    float w[NV][N];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int e = (i * L.lpr + L.sl) * N;
        if (p.weight && e < E) ld_weight<N>(p.weight, p.w_f32, g * E + e, w[i]);
        else {
#pragma unroll
            for (int j = 0; j < N; ++j) w[i][j] = 1.f;
        }
    }
    for (long long sg = L.wave; sg < p.nsg; sg += L.nwave) {
        const long long slot = sg * L.rpw + L.rw;
        const bool live = slot < p.nslot;
        float x[NV][N], gs[NV][N];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int e = (i * L.lpr + L.sl) * N;
            if (live && e < E) {
                Piece<T>::ld(p.x, slot * E + e, x[i]);
                if (p.gate_pos) Piece<T>::ld(p.gate, slot * E + e, gs[i]);
            } else {
#pragma unroll
                for (int j = 0; j < N; ++j) { x[i][j] = 0.f; gs[i][j] = 0.f; }
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if (p.gate_pos) gs[i][j] = sigmoid_f(gs[i][j]);
                if (pre) x[i][j] *= gs[i][j];
                ss += x[i][j] * x[i][j];
            }
        float unused = 0.f;
        group_sum(L, ss, unused, sred, buf);
        const float rs = p.cn / sqrtf(ss * p.inv_e + p.eps);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int e = (i * L.lpr + L.sl) * N;
            float o[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                o[j] = x[i][j] * rs * w[i][j];
                if (post) o[j] *= gs[i][j];
            }
            if (live && e < E) Piece<T>::st(p.o, slot * E + e, o);
        }
    }
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void normalize_bwd_kernel(NormArgs p) {
    constexpr int N = Piece<T>::N;
    const NormLane L(p);
    __shared__ float sred[16];
    int buf = 0;
    const bool pre = p.gate_pos == 1, post = p.gate_pos == 2, has_w = p.weight != nullptr;
    const int E = p.E;
    const int g = (int)((L.wave * L.rpw + L.rw) % p.G);
    float w[NV][N], dw[NV][N];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int e = (i * L.lpr + L.sl) * N;
        if (has_w && e < E) ld_weight<N>(p.weight, p.w_f32, g * E + e, w[i]);
        else {
#pragma unroll
            for (int j = 0; j < N; ++j) w[i][j] = 1.f;
        }
#pragma unroll
        for (int j = 0; j < N; ++j) dw[i][j] = 0.f;
    }
    for (long long sg = L.wave; sg < p.nsg; sg += L.nwave) {
        const long long slot = sg * L.rpw + L.rw;
        const bool live = slot < p.nslot;
        float x[NV][N], gs[NV][N], dr[NV][N];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int e = (i * L.lpr + L.sl) * N;
            if (live && e < E) {
                Piece<T>::ld(p.x, slot * E + e, x[i]);
                Piece<T>::ld(p.d_o, slot * E + e, dr[i]);
                if (p.gate_pos) Piece<T>::ld(p.gate, slot * E + e, gs[i]);
            } else {
#pragma unroll
                for (int j = 0; j < N; ++j) { x[i][j] = 0.f; gs[i][j] = 0.f; dr[i][j] = 0.f; }
            }
        }
        // x: the normalised quantity (gated when the gate comes first); dr: gradient of x / sigma before the weight
        float ss = 0.f, sd = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if (p.gate_pos) gs[i][j] = sigmoid_f(gs[i][j]);
                if (pre) x[i][j] *= gs[i][j];
                dr[i][j] *= p.cn;
                if (post) dr[i][j] *= gs[i][j];
                ss += x[i][j] * x[i][j];
                sd += x[i][j] * dr[i][j] * w[i][j];
            }
        group_sum(L, ss, sd, sred, buf);
        const float inv = 1.f / sqrtf(ss * p.inv_e + p.eps);          // 1 / sigma
        const float proj = sd * inv * p.inv_e;                         // sum(r * dr * w) / E, r = x / sigma
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int e = (i * L.lpr + L.sl) * N;
            float dx[N], dg[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                const float r = x[i][j] * inv;
                dw[i][j] += dr[i][j] * r;
                const float dxn = inv * (dr[i][j] * w[i][j] - r * proj);
                if (pre) {
                    // x = x_in * gs: d x_in = dxn * gs, d gate = dxn * x_in * gs (1 - gs) = dxn * x * (1 - gs)
                    dx[j] = dxn * gs[i][j];
                    dg[j] = dxn * x[i][j] * (1.f - gs[i][j]);
                } else if (post) {
                    // o = n * gs with n = cn * r * w; dr already carries gs, so d gate = do * n * gs (1 - gs)
                    dx[j] = dxn;
                    dg[j] = dr[i][j] * r * w[i][j] * (1.f - gs[i][j]);
                } else {
                    dx[j] = dxn;
                    dg[j] = 0.f;
                }
            }
            if (live && e < E) {
                Piece<T>::st(p.dx, slot * E + e, dx);
                if (p.gate_pos) Piece<T>::st(p.dgate, slot * E + e, dg);
            }
        }
    }
    if (has_w) {
        long long prow = L.wave * L.rpw + L.rw;
        if (p.wg_reduce) {
            // lane by lane the four wavefronts hold the same columns: waves 2, 3 hand over to 0, 1, then 1 to 0
            __shared__ float swg[2 * NV * N * 64];
            const int wl = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
            for (int round = 0; round < 2; ++round) {
                const int half = 2 >> round;                  // 2, then 1
                if (wl >= half && wl < 2 * half) {
#pragma unroll
                    for (int i = 0; i < NV; ++i)
#pragma unroll
                        for (int j = 0; j < N; ++j) swg[((wl - half) * NV * N + i * N + j) * 64 + lane] = dw[i][j];
                }
                __syncthreads();
                if (wl < half) {
#pragma unroll
                    for (int i = 0; i < NV; ++i)
#pragma unroll
                        for (int j = 0; j < N; ++j) dw[i][j] += swg[(wl * NV * N + i * N + j) * 64 + lane];
                }
                __syncthreads();
            }
            if (wl != 0) return;
            prow = (long long)blockIdx.x * L.rpw + L.rw;
        }
        float* row = p.partial + prow * E;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int e = (i * L.lpr + L.sl) * N;
            if (e < E) {
#pragma unroll
                for (int j = 0; j < N; j += 4) {
                    f32x4 v = {dw[i][j], dw[i][j + 1], dw[i][j + 2], dw[i][j + 3]};
                    *reinterpret_cast<f32x4*>(row + e + j) = v;
                }
            }
        }
    }
}

// dw[g*E + e] = sum of the partial rows idx = g, g + G, g + 2G, ... ; one workgroup per 16 columns: 4 lanes of four
// columns each, 64 row phases, summed through LDS in a fixed order.
__global__ __launch_bounds__(256) void normalize_dw_kernel(const float* __restrict__ partial, float* __restrict__ dw,
                                                           long long nrow, int G, int E) {
    __shared__ f32x4 red[64][4];
    const int cq = threadIdx.x & 3, rl = threadIdx.x >> 2;
    const long long col = (long long)blockIdx.x * 16 + cq * 4;
    const long long D = (long long)G * E;
    f32x4 acc = zero4();
    if (col < D) {
        const int g = (int)(col / E), e = (int)(col % E);
        for (long long idx = g + (long long)rl * G; idx < nrow; idx += 64LL * G)
            acc += *reinterpret_cast<const f32x4*>(partial + idx * E + e);
    }
    red[rl][cq] = acc;
    __syncthreads();
    if (rl == 0 && col < D) {
        f32x4 s = red[0][cq];
#pragma unroll
        for (int r = 1; r < 64; ++r) s += red[r][cq];
        *reinterpret_cast<f32x4*>(dw + col) = s;
    }
}

// Launch shape shared by both passes and by the workspace size.
struct NormCfg {
    int n, nv, lpr_log2, rpw, wg_reduce, wg_row;
    long long nslot, nsg, nwg;
    long long partial_rows() const { return wg_row ? nwg : nwg * (wg_reduce ? 1 : 4) * rpw; }
};

static long long gcd_ll(long long a, long long b) { while (b) { const long long t = a % b; a = b; b = t; } return a; }

static int norm_config(const hdla_norm_dims* d, bool bwd, NormCfg& c) {
    if (!d) return HDLA_ERR_NULL;
    if (d->dtype != HDLA_BF16 && d->dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    if (d->weight_dtype != HDLA_BF16 && d->weight_dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    if (d->gate_pos < 0 || d->gate_pos > 2) return HDLA_ERR_SHAPE;
    if (d->rows < 0 || d->G <= 0 || d->E <= 0 || !(d->eps >= 0.f)) return HDLA_ERR_SHAPE;
    c.n = d->dtype == HDLA_BF16 ? 8 : 4;
    if (d->E % c.n) return HDLA_ERR_SHAPE;                      // groups start on 16-byte boundaries
    const int pieces = d->E / c.n;
    if (pieces > 256 * 8) return HDLA_ERR_SHAPE;                // a group lives in one workgroup's registers
    if (d->rows > (1LL << 40) / d->G) return HDLA_ERR_SHAPE;
    c.nslot = d->rows * d->G;
    // long groups always, and groups of at least 128 pieces when there are too few of them to fill the chip one
    // wavefront each (a decode step: a few hundred rows)
    c.wg_row = pieces > 64 * 8 || (pieces >= 128 && c.nslot <= 2048);
    if (c.wg_row) {
        // one group per workgroup pass, 256 lanes across it
        c.nv = 1;
        while (c.nv * 256 < pieces) c.nv *= 2;
        c.lpr_log2 = 8; c.rpw = 1; c.wg_reduce = 0;
        c.nsg = c.nslot;
    } else {
        c.nv = 1;
        while (c.nv * 64 < pieces) c.nv *= 2;
        const int per = (pieces + c.nv - 1) / c.nv;
        c.lpr_log2 = 0;
        while ((1 << c.lpr_log2) < per) ++c.lpr_log2;
        c.rpw = 64 >> c.lpr_log2;
        c.nsg = (c.nslot + c.rpw - 1) / c.rpw;
        c.wg_reduce = c.rpw % d->G == 0;
    }
    // a few passes per wavefront to amortise the weight loads, enough workgroups to fill the chip, and, backward, a
    // bound on the partial rows of the weight gradient; then a multiple of what keeps a lane on one weight column
    const long long cap = bwd ? 1024 : 8192, owners = c.wg_row ? 1 : 4;
    const long long per_wave = c.nsg >= 4 * owners * 1024 ? 4 : (c.nsg >= 2 * owners * 1024 ? 2 : 1);
    long long nwg = (c.nsg + owners * per_wave - 1) / (owners * per_wave);
    if (nwg < 1) nwg = 1;
    if (nwg > cap) nwg = cap;
    const long long m = d->G / gcd_ll(d->G, owners * c.rpw);
    if (m > 65536) return HDLA_ERR_SHAPE;
    c.nwg = (nwg + m - 1) / m * m;
    return HDLA_OK;
}

template <typename T>
static hipError_t launch_norm(const NormArgs& a, const NormCfg& c, bool bwd, hipStream_t s) {
    const dim3 grid((unsigned)c.nwg), block(256);
#define HDLA_NORM_CASE(NVV)                                                                              \
    case NVV:                                                                                            \
        if (bwd) hipLaunchKernelGGL((normalize_bwd_kernel<T, NVV>), grid, block, 0, s, a);               \
        else hipLaunchKernelGGL((normalize_fwd_kernel<T, NVV>), grid, block, 0, s, a);                   \
        break;
    switch (c.nv) {
        HDLA_NORM_CASE(1)
        HDLA_NORM_CASE(2)
        HDLA_NORM_CASE(4)
        HDLA_NORM_CASE(8)
        default: return hipErrorInvalidValue;
    }
#undef HDLA_NORM_CASE
    return hipGetLastError();
}

static NormArgs norm_args(const hdla_norm_dims* d, const NormCfg& c) {
    NormArgs a{};
    a.nslot = c.nslot; a.nsg = c.nsg; a.G = d->G; a.E = d->E; a.lpr_log2 = c.lpr_log2;
    a.w_f32 = d->weight_dtype == HDLA_FP32; a.gate_pos = d->gate_pos; a.wg_reduce = c.wg_reduce; a.wg_row = c.wg_row;
    a.cn = d->c / sqrtf((float)d->E); a.inv_e = 1.f / (float)d->E; a.eps = d->eps;
    return a;
}

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace hdla

using namespace hdla;

extern "C" size_t hdla_normalize_workspace_bytes(const hdla_norm_dims* dims) {
    NormCfg c;
    if (norm_config(dims, true, c) != HDLA_OK) return 0;
    return (size_t)c.partial_rows() * dims->E * sizeof(float);
}

extern "C" int hdla_normalize_fwd(const hdla_norm_dims* dims, const void* x, const void* weight, const void* gate,
                                  void* o, void* stream) {
    NormCfg c;
    const int rc = norm_config(dims, false, c);
    if (rc) return rc;
    if (dims->rows == 0) return HDLA_OK;
    if (!x || !o || (dims->gate_pos && !gate)) return HDLA_ERR_NULL;
    if (!al16(x) || !al16(o) || !al16(gate) || !al16(weight)) return HDLA_ERR_ALIGN;
    NormArgs a = norm_args(dims, c);
    a.x = x; a.weight = weight; a.gate = gate; a.o = o;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = dims->dtype == HDLA_BF16 ? launch_norm<bf16>(a, c, false, s) : launch_norm<float>(a, c, false, s);
    return e == hipSuccess ? HDLA_OK : (int)e;
}

extern "C" int hdla_normalize_bwd(const hdla_norm_dims* dims, const void* x, const void* weight, const void* gate,
                                  const void* d_o, void* dx, void* dgate, float* dw, void* workspace,
                                  size_t workspace_bytes, void* stream) {
    NormCfg c;
    const int rc = norm_config(dims, true, c);
    if (rc) return rc;
    if (weight && !dw) return HDLA_ERR_NULL;
    if (dims->rows > 0 && (!x || !d_o || !dx || (dims->gate_pos && (!gate || !dgate)))) return HDLA_ERR_NULL;
    if (!al16(x) || !al16(d_o) || !al16(dx) || !al16(gate) || !al16(dgate) || !al16(weight) || !al16(dw))
        return HDLA_ERR_ALIGN;
    const size_t need = weight ? (size_t)c.partial_rows() * dims->E * sizeof(float) : 0;
    if (need && (!workspace || !al16(workspace) || workspace_bytes < need)) return HDLA_ERR_WORKSPACE;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    NormArgs a = norm_args(dims, c);
    a.x = x; a.weight = weight; a.gate = gate; a.d_o = d_o; a.dx = dx; a.dgate = dgate;
    a.partial = static_cast<float*>(workspace);
    if (dims->rows > 0) {
        const hipError_t e = dims->dtype == HDLA_BF16 ? launch_norm<bf16>(a, c, true, s) : launch_norm<float>(a, c, true, s);
        if (e != hipSuccess) return (int)e;
    }
    if (weight) {
        const long long D = (long long)dims->G * dims->E;
        hipLaunchKernelGGL(normalize_dw_kernel, dim3((unsigned)((D + 15) / 16)), dim3(256), 0, s, a.partial, dw,
                           dims->rows > 0 ? c.partial_rows() : 0LL, dims->G, dims->E);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
    return HDLA_OK;
}
