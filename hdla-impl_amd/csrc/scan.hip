// The two inter-chunk state scans: the only sequential part of the chunked operator.
//
// scan_fwd replaces HRDPLR/fwd_triton.py:808-968 (state recurrence, h checkpoints, v_new, final state) and, in
// the forward pass, also HRDPLR/fwd_triton.py:984-1095 (the output o), so the forward pass never writes h.
// scan_bwd replaces HRDPLR/bwd_triton.py:127-222 (reverse recurrence of the state gradient, dh checkpoints,
// dh0) fused with the dv_new part of HRDPLR/bwd_triton.py:30-105.
//
// One wavefront owns a K x 16 column block of the fp32 state of one (sequence, head) for the whole sequence;
// one single-wave workgroup each, numbered so that the blocks of one (sequence, head) share an XCD's L2.
// The block lives in MFMA accumulators as the row fragment of S^T (rows = value column, inner = channel), which
// is at once the operand layout of the next product: w S, qg S and the rank updates chain through registers
// with no LDS traffic and no cross-lane movement.  All per-chunk operands were written by the prep kernel in
// fragment order, so each is one coalesced 512-byte (bf16) load per tile; the loads of the next few chunks are
// in flight while one chunk is computed.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

// ---- block numbering ------------------------------------------------------------------------------------------
// The V/16 column blocks of one (sequence, head) read the same w/kg/bg/qg tiles.  Workgroups are handed to the
// eight XCDs round-robin by their linear index and each XCD has its own L2, so the linear index is decoded as
// (pair mod 8) + 8 * (column block + V/16 * (pair / 8)): all column blocks of a pair land on one XCD (shared
// tiles come from HBM once per pair instead of V/16 times) but on different compute units (each wave keeps a
// whole register file and its own L1 bandwidth).
constexpr int XCDS = 8;
static inline unsigned scan_grid(int H, int N, int VT) { return (unsigned)(XCDS * VT * ((H * N + XCDS - 1) / XCDS)); }
template <typename T>
__device__ __forceinline__ bool scan_block(const ChunkArgs<T>& p, int VT, int& vt, int& h, int& n) {
    const int L = blockIdx.x, xcd = L % XCDS, idx = L / XCDS;
    vt = idx % VT;
    const int pair = (idx / VT) * XCDS + xcd;
    if (pair >= p.H * p.st.N) return false;
    n = pair / p.H;
    h = pair - n * p.H;
    return true;
}

// ---- forward -------------------------------------------------------------------------------------------------
template <typename T, int K, int V, bool WRITE_O>
struct FwdOps {
    static constexpr int KT = K / 16;
    Frag<T> w[2][KT], kgt[KT], bgt[2][KT], ut[2], vtt;
    Frag<T> qg[WRITE_O ? KT : 1], aqk, aqb[2];
    f32x4 egl[KT];

    __device__ __forceinline__ void load(const Ws<T>& ws, int64_t chw, int vt) {
        constexpr int VT = V / 16, KT2 = KT / 2;
        const int l = lane_id(), g = l >> 4;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            ld_pair(ws.W + ((chw * 2 + 0) * KT2 + kp) * PAIR, w[0][2 * kp], w[0][2 * kp + 1]);
            ld_pair(ws.W + ((chw * 2 + 1) * KT2 + kp) * PAIR, w[1][2 * kp], w[1][2 * kp + 1]);
            ld_pair(ws.KGT + (chw * KT2 + kp) * PAIR, kgt[2 * kp], kgt[2 * kp + 1]);
            ld_pair(ws.BGT + ((chw * 2 + 0) * KT2 + kp) * PAIR, bgt[0][2 * kp], bgt[0][2 * kp + 1]);
            ld_pair(ws.BGT + ((chw * 2 + 1) * KT2 + kp) * PAIR, bgt[1][2 * kp], bgt[1][2 * kp + 1]);
            if (WRITE_O) ld_pair(ws.QG + (chw * KT2 + kp) * PAIR, qg[2 * kp], qg[2 * kp + 1]);
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) egl[kt] = *reinterpret_cast<const f32x4*>(ws.EGL + chw * K + 16 * kt + 4 * g);
        ld_pair(ws.UT + (chw * VT + vt) * PAIR, ut[0], ut[1]);
        vtt = ld_tile(ws.VTT + (chw * VT + vt) * TILE);
        if (WRITE_O) {
            aqk = ld_tile(ws.AQK + chw * TILE);
            ld_pair(ws.AQB + chw * PAIR, aqb[0], aqb[1]);
        }
    }
};

template <typename T, int K, int V, bool WRITE_O>
__global__ __launch_bounds__(64) void scan_fwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16;
    int vt, h, n;
    if (!scan_block(p, V / 16, vt, h, n)) return;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int blk = blockIdx.x;
    PHASE_CLOCK(p, blk, 0);

    // state block: lane (g,c) reg i of tile kt = S[16kt + 4g + i][16vt + c]
    f32x4 S[KT];
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) S[kt] = zero4();
    if (p.h0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) S[kt][i] = p.h0[soff + (int64_t)(16 * kt + 4 * g + i) * V];
    }

    // Operand sets of the next NBUF-1 chunks are in flight while one chunk is computed: each step of the scan
    // would otherwise wait a full memory round trip.  NBUF is what the register file holds without spilling.
    constexpr int NBUF = sizeof(T) == 2 ? (K == 64 ? 4 : 2) : (K == 64 ? 2 : 1);
    FwdOps<T, K, V, WRITE_O> buf[NBUF];
    const Frag<T> ident = ident_frag<T>();
    const int64_t chw0 = (int64_t)h * p.st.nch;

    auto step = [&](const FwdOps<T, K, V, WRITE_O>& cur, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + cid;
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        Frag<T> sb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sb[kt] = to_frag<T>(S[kt]);
        if (!WRITE_O) {
            // checkpoint of the entering state, row-major [K][V]: one transposing product per tile turns the
            // register layout (4 channels of one value column per lane) into 4 consecutive values of one channel
            T* hc = p.ws.HC + chw * (K * V) + 16 * vt + 4 * g;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) st_frag(hc + (16 * kt + c) * V, transpose(sb[kt], ident));
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
            T* vnp = p.ws.VN + chw * (2 * CH * V) + 16 * vt + 4 * g;
#pragma unroll
            for (int s = 0; s < 2; ++s) st_frag(vnp + (s * CH + c) * V, transpose(vnb[s], ident));
        }
        if (WRITE_O) {
            // o (rows token, inner value) = qg S + A_qk v + sum_s A_qb^s v_new_s
            f32x4 o = zero4();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) o = mm(cur.qg[kt], sb[kt], o);
            o = mm(cur.aqk, cur.vtt, o);
            o = mm(cur.aqb[0], vnb[0], o);
            o = mm(cur.aqb[1], vnb[1], o);
            if (c < len) st_frag(p.o + ((tok0 + c) * H + h) * V + 16 * vt + 4 * g, to_frag<T>(o));
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
    };

    // Every load of the main loop is unconditional (prefetch indices are clamped to the last chunk): a load or
    // store that may or may not have been issued would force the compiler to wait for all outstanding memory
    // operations instead of only those of the oldest operand set.
    const int nfull = (c1 - c0) / NBUF;
    if (c0 < c1) {
#pragma unroll
        for (int j = 0; j < NBUF - 1; ++j) buf[j].load(p.ws, chw0 + min(c0 + j, c1 - 1), vt);
#pragma unroll 1
        for (int gi = 0; gi < nfull; ++gi) {
            const int base = c0 + gi * NBUF;
#pragma unroll
            for (int j = 0; j < NBUF; ++j) {
                buf[(j + NBUF - 1) % NBUF].load(p.ws, chw0 + min(base + j + NBUF - 1, c1 - 1), vt);
                step(buf[j], base + j);
            }
        }
#pragma unroll 1
        for (int cid = c0 + nfull * NBUF; cid < c1; ++cid) {      // fewer than NBUF chunks left
            buf[0].load(p.ws, chw0 + cid, vt);
            step(buf[0], cid);
        }
    }
    PHASE_CLOCK(p, blk, 1);
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

    __device__ __forceinline__ void load(const ChunkArgs<T>& p, int cid, int c0, int64_t bos, int64_t eos, int h, int vt) {
        constexpr int KT2 = KT / 2;
        const int l = lane_id(), g = l >> 4, c = l & 15;
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        const Ws<T>& ws = p.ws;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            ld_pair(ws.BG + ((chw * 2 + 0) * KT2 + kp) * PAIR, bg[0][2 * kp], bg[0][2 * kp + 1]);
            ld_pair(ws.BG + ((chw * 2 + 1) * KT2 + kp) * PAIR, bg[1][2 * kp], bg[1][2 * kp + 1]);
            ld_pair(ws.WT + ((chw * 2 + 0) * KT2 + kp) * PAIR, wt[0][2 * kp], wt[0][2 * kp + 1]);
            ld_pair(ws.WT + ((chw * 2 + 1) * KT2 + kp) * PAIR, wt[1][2 * kp], wt[1][2 * kp + 1]);
            ld_pair(ws.QGT + (chw * KT2 + kp) * PAIR, qgt[2 * kp], qgt[2 * kp + 1]);
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) egl[kt] = *reinterpret_cast<const f32x4*>(ws.EGL + chw * K + 16 * kt + 4 * g);
        ld_pair(ws.AQBT + chw * PAIR, aqbt[0], aqbt[1]);
        // rows past the end of a ragged chunk alias its last row here and are zeroed where the value is used:
        // a select right after the load would make the wave wait for this (youngest) load at once
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        don = ld_frag(p.dout + ((tok0 + min(c, len - 1)) * p.H + h) * V + 16 * vt + 4 * g);
    }
};

template <typename T, int K, int V>
__global__ __launch_bounds__(64) void scan_bwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16;
    int vt, h, n;
    if (!scan_block(p, V / 16, vt, h, n)) return;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int blk = blockIdx.x;
    PHASE_CLOCK(p, blk, 0);

    f32x4 dS[KT];   // lane (g,c) reg i of tile kt = dS[16kt + 4g + i][16vt + c]
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) dS[kt] = zero4();
    if (p.dht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) dS[kt][i] = p.dht[soff + (int64_t)(16 * kt + 4 * g + i) * V];
    }
    const Frag<T> ident = ident_frag<T>();

    constexpr int NBUF = sizeof(T) == 2 ? (K == 64 ? 4 : 2) : (K == 64 ? 2 : 1);
    BwdOps<T, K, V> buf[NBUF];

    auto step = [&](const BwdOps<T, K, V>& cur, int cid) __attribute__((always_inline)) {
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        Frag<T> dsb[KT];
        T* dhc = p.ws.DHC + chw * (K * V) + 16 * vt + 4 * g;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            dsb[kt] = to_frag<T>(dS[kt]);
            st_frag(dhc + (16 * kt + c) * V, transpose(dsb[kt], ident));     // row-major [K][V], 8-byte stores
        }
        const int len = (int)min((int64_t)CH, eos - (bos + (int64_t)(cid - c0) * CH));
        Frag<T> don = cur.don;
        if (c >= len) don = zero_frag<T>();
        const Frag<T> doT = transpose(don, ident);          // rows value, inner token
        // dv_new_s^T (rows value, inner token) = do^T A_qb^s + dS^T bg_s^T
        f32x4 dvn[2];
        dvn[0] = mm(doT, cur.aqbt[0], zero4());
        dvn[1] = mm(doT, cur.aqbt[1], zero4());
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            dvn[0] = mm(dsb[kt], cur.bg[0][kt], dvn[0]);
            dvn[1] = mm(dsb[kt], cur.bg[1][kt], dvn[1]);
        }
        const Frag<T> dvb[2] = {to_frag<T>(dvn[0]), to_frag<T>(dvn[1])};
        T* dvp = p.ws.DVN + chw * (2 * CH * V) + 16 * vt + 4 * g;
#pragma unroll
        for (int s = 0; s < 2; ++s) st_frag(dvp + (s * CH + c) * V, transpose(dvb[s], ident));
        // dS <- exp(g_last) dS + qg^T do + sum_s w_s^T dv_new_s
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 x = dS[kt] * cur.egl[kt];
            x = mm(doT, cur.qgt[kt], x);
            x = mm(dvb[0], cur.wt[0][kt], x);
            x = mm(dvb[1], cur.wt[1][kt], x);
            dS[kt] = x;
        }
    };

    const int nfull = (c1 - c0) / NBUF;
    if (c0 < c1) {
#pragma unroll
        for (int j = 0; j < NBUF - 1; ++j) buf[j].load(p, max(c1 - 1 - j, c0), c0, bos, eos, h, vt);
#pragma unroll 1
        for (int gi = 0; gi < nfull; ++gi) {
            const int base = c1 - 1 - gi * NBUF;
#pragma unroll
            for (int j = 0; j < NBUF; ++j) {
                buf[(j + NBUF - 1) % NBUF].load(p, max(base - j - (NBUF - 1), c0), c0, bos, eos, h, vt);
                step(buf[j], base - j);
            }
        }
#pragma unroll 1
        for (int cid = c1 - 1 - nfull * NBUF; cid >= c0; --cid) {
            buf[0].load(p, cid, c0, bos, eos, h, vt);
            step(buf[0], cid);
        }
    }
    PHASE_CLOCK(p, blk, 1);
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
    dim3 grid(scan_grid(a.H, a.st.N, V / 16)), block(64);
    if (write_o) hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}
template <typename T, int K, int V>
static hipError_t launch_scan_bwd_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(scan_grid(a.H, a.st.N, V / 16)), block(64);
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
