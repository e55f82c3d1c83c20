// The two inter-chunk state scans: the only sequential part of the chunked operator.
//
// scan_fwd replaces HRDPLR/fwd_triton.py:808-968 (state recurrence, h checkpoints, v_new, final state) and, in
// the forward pass, also HRDPLR/fwd_triton.py:984-1095 (the output o), so the forward pass never writes h.
// scan_bwd replaces HRDPLR/bwd_triton.py:127-222 (reverse recurrence of the state gradient, dh checkpoints,
// dh0) fused with the dv_new part of HRDPLR/bwd_triton.py:30-105.
//
// One wavefront owns a K x 16 column block of the fp32 state of one (sequence, head) for the whole sequence.
// The block lives in MFMA accumulators as the row fragment of S^T (rows = value column, inner = channel), which
// is at once the operand layout of the next product: w S, qg S and the rank updates chain through registers
// with no LDS traffic and no cross-lane movement.  All per-chunk operands were written by the prep kernel in
// fragment order, so each is one coalesced 512-byte (bf16) load per tile; the loads of chunk c+1 are issued
// before the products of chunk c.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

// ---- forward -------------------------------------------------------------------------------------------------
template <typename T, int K, int V, bool WRITE_O>
struct FwdOps {
    static constexpr int KT = K / 16;
    Frag<T> w[2][KT], kgt[KT], bgt[2][KT], ut[2], vtt;
    Frag<T> qg[WRITE_O ? KT : 1], aqk, aqb[2];
    f32x4 egl[KT];

    __device__ __forceinline__ void load(const Ws<T>& ws, int64_t chw, int vt) {
        constexpr int VT = V / 16;
        const int l = lane_id(), g = l >> 4;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            w[0][kt] = ld_tile(ws.W + ((chw * 2 + 0) * KT + kt) * TILE);
            w[1][kt] = ld_tile(ws.W + ((chw * 2 + 1) * KT + kt) * TILE);
            kgt[kt] = ld_tile(ws.KGT + (chw * KT + kt) * TILE);
            bgt[0][kt] = ld_tile(ws.BGT + ((chw * 2 + 0) * KT + kt) * TILE);
            bgt[1][kt] = ld_tile(ws.BGT + ((chw * 2 + 1) * KT + kt) * TILE);
            egl[kt] = *reinterpret_cast<const f32x4*>(ws.EGL + chw * K + 16 * kt + 4 * g);
            if (WRITE_O) qg[kt] = ld_tile(ws.QG + (chw * KT + kt) * TILE);
        }
        ut[0] = ld_tile(ws.UT + ((chw * 2 + 0) * VT + vt) * TILE);
        ut[1] = ld_tile(ws.UT + ((chw * 2 + 1) * VT + vt) * TILE);
        vtt = ld_tile(ws.VTT + (chw * VT + vt) * TILE);
        if (WRITE_O) {
            aqk = ld_tile(ws.AQK + chw * TILE);
            aqb[0] = ld_tile(ws.AQB + (chw * 2 + 0) * TILE);
            aqb[1] = ld_tile(ws.AQB + (chw * 2 + 1) * TILE);
        }
    }
};

template <typename T, int K, int V, bool WRITE_O>
__global__ __launch_bounds__(64) void scan_fwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16;
    const int vt = blockIdx.x, h = blockIdx.y, n = blockIdx.z;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);

    // state block: lane (g,c) reg i of tile kt = S[16kt + 4g + i][16vt + c]
    f32x4 S[KT];
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) S[kt][i] = p.h0 ? p.h0[soff + (int64_t)(16 * kt + 4 * g + i) * V] : 0.f;
    }

    // Operands of chunk c+1 are fetched while chunk c is computed when two sets fit the register file
    // (bf16 operands, or fp32 with K = 64); otherwise one set is loaded per step.
    constexpr bool PF = sizeof(T) == 2 || K == 64;
    FwdOps<T, K, V, WRITE_O> cur, nxt;
    if (PF && c0 < c1) cur.load(p.ws, (int64_t)h * p.st.nch + c0, vt);
#pragma unroll 1
    for (int cid = c0; cid < c1; ++cid) {
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        if (PF) { if (cid + 1 < c1) nxt.load(p.ws, chw + 1, vt); }
        else cur.load(p.ws, chw, vt);
        ChunkPos cp;
        locate_chunk(p.st, cid, cp);

        Frag<T> sb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sb[kt] = to_frag<T>(S[kt]);
        if (!WRITE_O) {
            T* hc = p.ws.HC + chw * (K * V) + 16 * vt + c;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) st_elem(hc + (16 * kt + 4 * g + i) * V, S[kt][i]);
        }
        // v_new^T (rows value, inner token) = u^T + S^T w^T
        f32x4 vn[2] = {to_f32(cur.ut[0]), to_f32(cur.ut[1])};
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            vn[0] = mm(sb[kt], cur.w[0][kt], vn[0]);
            vn[1] = mm(sb[kt], cur.w[1][kt], vn[1]);
        }
        const Frag<T> vnb[2] = {to_frag<T>(vn[0]), to_frag<T>(vn[1])};
        if (!WRITE_O) {
            T* vnp = p.ws.VN + chw * (2 * CH * V) + 16 * vt + c;
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) st_elem(vnp + (s * CH + 4 * g + i) * V, vn[s][i]);
        }
        if (WRITE_O) {
            // o (rows token, inner value) = qg S + A_qk v + sum_s A_qb^s v_new_s
            f32x4 o = zero4();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) o = mm(cur.qg[kt], sb[kt], o);
            o = mm(cur.aqk, cur.vtt, o);
            o = mm(cur.aqb[0], vnb[0], o);
            o = mm(cur.aqb[1], vnb[1], o);
            if (c < cp.len) st_frag(p.o + ((cp.tok0 + c) * H + h) * V + 16 * vt + 4 * g, to_frag<T>(o));
        }
        // S <- exp(g_last) S + kg^T v + sum_s bg_s^T v_new_s
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 x = S[kt] * cur.egl[kt];
            x = mm(cur.vtt, cur.kgt[kt], x);
            x = mm(vnb[0], cur.bgt[0][kt], x);
            x = mm(vnb[1], cur.bgt[1][kt], x);
            S[kt] = x;
        }
        if (PF) cur = nxt;
    }
    if (p.ht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
template <typename T, int K, int V>
struct BwdOps {
    static constexpr int KT = K / 16;
    Frag<T> aqbt[2], bg[2][KT], wt[2][KT], qgt[KT], don;
    f32x4 egl[KT];

    __device__ __forceinline__ void load(const ChunkArgs<T>& p, int cid, int h, int vt) {
        const int l = lane_id(), g = l >> 4, c = l & 15;
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        const Ws<T>& ws = p.ws;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            bg[0][kt] = ld_tile(ws.BG + ((chw * 2 + 0) * KT + kt) * TILE);
            bg[1][kt] = ld_tile(ws.BG + ((chw * 2 + 1) * KT + kt) * TILE);
            wt[0][kt] = ld_tile(ws.WT + ((chw * 2 + 0) * KT + kt) * TILE);
            wt[1][kt] = ld_tile(ws.WT + ((chw * 2 + 1) * KT + kt) * TILE);
            qgt[kt] = ld_tile(ws.QGT + (chw * KT + kt) * TILE);
            egl[kt] = *reinterpret_cast<const f32x4*>(ws.EGL + chw * K + 16 * kt + 4 * g);
        }
        aqbt[0] = ld_tile(ws.AQBT + (chw * 2 + 0) * TILE);
        aqbt[1] = ld_tile(ws.AQBT + (chw * 2 + 1) * TILE);
        ChunkPos cp;
        locate_chunk(p.st, cid, cp);
        don = ld_frag_if(p.dout + ((cp.tok0 + c) * p.H + h) * V + 16 * vt + 4 * g, c < cp.len);
    }
};

template <typename T, int K, int V>
__global__ __launch_bounds__(64) void scan_bwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16;
    const int vt = blockIdx.x, h = blockIdx.y, n = blockIdx.z;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);

    f32x4 dS[KT];   // lane (g,c) reg i of tile kt = dS[16kt + 4g + i][16vt + c]
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) dS[kt][i] = p.dht ? p.dht[soff + (int64_t)(16 * kt + 4 * g + i) * V] : 0.f;
    }
    const Frag<T> ident = ident_frag<T>();

    constexpr bool PF = sizeof(T) == 2 || K == 64;
    BwdOps<T, K, V> cur, nxt;
    if (PF && c0 < c1) cur.load(p, c1 - 1, h, vt);
#pragma unroll 1
    for (int cid = c1 - 1; cid >= c0; --cid) {
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        if (PF) { if (cid > c0) nxt.load(p, cid - 1, h, vt); }
        else cur.load(p, cid, h, vt);

        Frag<T> dsb[KT];
        T* dhc = p.ws.DHC + chw * (K * V) + 16 * vt + c;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            dsb[kt] = to_frag<T>(dS[kt]);
#pragma unroll
            for (int i = 0; i < 4; ++i) st_elem(dhc + (16 * kt + 4 * g + i) * V, dS[kt][i]);
        }
        const Frag<T> doT = transpose(cur.don, ident);      // rows value, inner token
        // dv_new_s^T (rows value, inner token) = do^T A_qb^s + dS^T bg_s^T
        f32x4 dvn[2];
        dvn[0] = mm(doT, cur.aqbt[0], zero4());
        dvn[1] = mm(doT, cur.aqbt[1], zero4());
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            dvn[0] = mm(dsb[kt], cur.bg[0][kt], dvn[0]);
            dvn[1] = mm(dsb[kt], cur.bg[1][kt], dvn[1]);
        }
        T* dvp = p.ws.DVN + chw * (2 * CH * V) + 16 * vt + c;
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) st_elem(dvp + (s * CH + 4 * g + i) * V, dvn[s][i]);
        const Frag<T> dvb[2] = {to_frag<T>(dvn[0]), to_frag<T>(dvn[1])};
        // dS <- exp(g_last) dS + qg^T do + sum_s w_s^T dv_new_s
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 x = dS[kt] * cur.egl[kt];
            x = mm(doT, cur.qgt[kt], x);
            x = mm(dvb[0], cur.wt[0][kt], x);
            x = mm(dvb[1], cur.wt[1][kt], x);
            dS[kt] = x;
        }
        if (PF) cur = nxt;
    }
    if (p.dh0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.dh0[soff + (int64_t)(16 * kt + 4 * g + i) * V] = dS[kt][i];
    }
}

// ---- launchers -----------------------------------------------------------------------------------------------
template <typename T, int K, int V>
static hipError_t launch_scan_fwd_kv(const ChunkArgs<T>& a, bool write_o, hipStream_t stream) {
    dim3 grid(V / 16, a.H, a.st.N), block(64);
    if (write_o) hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}
template <typename T, int K, int V>
static hipError_t launch_scan_bwd_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(V / 16, a.H, a.st.N), block(64);
    hipLaunchKernelGGL((scan_bwd_kernel<T, K, V>), grid, block, 0, stream, a);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_scan_fwd(const ChunkArgs<T>& a, int K, int V, bool write_o, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_scan_fwd_kv<T, 64, 64>(a, write_o, stream);
    if (K == 128 && V == 128) return launch_scan_fwd_kv<T, 128, 128>(a, write_o, stream);
    if (K == 64 && V == 128) return launch_scan_fwd_kv<T, 64, 128>(a, write_o, stream);
    if (K == 128 && V == 64) return launch_scan_fwd_kv<T, 128, 64>(a, write_o, stream);
    return hipErrorInvalidValue;
}
template <typename T>
hipError_t launch_scan_bwd(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_scan_bwd_kv<T, 64, 64>(a, stream);
    if (K == 128 && V == 128) return launch_scan_bwd_kv<T, 128, 128>(a, stream);
    if (K == 64 && V == 128) return launch_scan_bwd_kv<T, 64, 128>(a, stream);
    if (K == 128 && V == 64) return launch_scan_bwd_kv<T, 128, 64>(a, stream);
    return hipErrorInvalidValue;
}
template hipError_t launch_scan_fwd<bf16>(const ChunkArgs<bf16>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_fwd<float>(const ChunkArgs<float>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_bwd<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_scan_bwd<float>(const ChunkArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
