// The two inter-chunk state scans: the only sequential part of the chunked operator.
//
// scan_fwd replaces HRDPLR/fwd_triton.py:808-968 (state recurrence, h checkpoints, v_new, final state) and, in
// the forward pass, also HRDPLR/fwd_triton.py:984-1095 (the output o), so the forward pass never writes h.
// scan_bwd replaces HRDPLR/bwd_triton.py:127-222 (reverse recurrence of the state gradient, dh checkpoints,
// dh0) fused with the dv_new part of HRDPLR/bwd_triton.py:30-105.
//
// One workgroup per (sequence, head), one wavefront per 16-column block of the fp32 state.  A wave keeps its
// K x 16 block in MFMA accumulators as the row fragment of S^T (rows = value column, inner = channel), which is
// at once the operand layout of the next product: w S, qg S and the rank updates chain through registers with
// no cross-lane movement.
//
// What bounds a step is not arithmetic but operand delivery: a wave may have at most 63 memory instructions in
// flight, and every wave of a head needs the same w / kg / bg / qg tiles.  So the waves of a workgroup split the
// chunk's shared operand block (one contiguous block per chunk, written by the prep kernel) between them:
// each wave fetches its share of the block of chunk c+6 into registers (16 bytes per lane, a few instructions),
// hands the share of chunk c+1 to LDS, and all waves read the operands of chunk c from LDS.  One LDS-only
// barrier per chunk; global loads stay in flight across it.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// workgroup barrier that orders LDS accesses only: global loads issued before it may still be outstanding
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// depth of the register ring of operand shares: enough chunks in flight to cover the memory latency
template <typename T, int K, int V> struct ScanCfg {
    static constexpr int NW = V / 16;                                            // wavefronts per workgroup
    static constexpr int DR = (sizeof(T) == 2 && NW == 4 && K == 64) ? 6 : (sizeof(T) == 2 || K == 64) ? 4 : 2;
    // whether the ring also carries the wave's own u and v tiles; the largest fp32 shape has no registers left
    // for them and loads them where they are used
    static constexpr bool RING_OWN = !(sizeof(T) == 4 && K == 128 && V == 128);
    // When a step reads its shared operands from LDS.  2: all of them before the first product; 1: those of the
    // state update only once the products of v_new are issued; 0: wherever the compiler puts them (shapes whose
    // registers allow nothing else).  KB = bytes of one operand row; with_o = the scan also produces the output.
    static constexpr int read_mode(bool with_o) {
        constexpr int KB = K * (int)sizeof(T);
        if (KB <= 128) return 2;
        if (KB >= 512 || (V == 128 && with_o)) return 0;
        return 1;
    }
};

// one wave's share of a shared operand block: instructions w, w+NW, ... of the NI 1-KiB pieces
template <int NI, int NW> struct Share {
    static constexpr int CNT = (NI + NW - 1) / NW;
    i32x4 a[CNT];
    __device__ __forceinline__ void load(const char* blk, int w) {
        const int l = lane_id();
#pragma unroll
        for (int j = 0; j < CNT; ++j) {
            const int i = min(w + j * NW, NI - 1);        // the last pieces may be fetched twice; never out of range
            a[j] = *reinterpret_cast<const i32x4*>(blk + i * 1024 + l * 16);
        }
    }
    __device__ __forceinline__ void to_lds(char* slot, int w) const {
        const int l = lane_id();
#pragma unroll
        for (int j = 0; j < CNT; ++j) {
            const int i = min(w + j * NW, NI - 1);
            *reinterpret_cast<i32x4*>(slot + i * 1024 + l * 16) = a[j];
        }
    }
};

// ---- forward -------------------------------------------------------------------------------------------------
template <typename T, int K, int V, bool WRITE_O>
__global__ __launch_bounds__(V * 4) void scan_fwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NW = ScanCfg<T, K, V>::NW, DR = ScanCfg<T, K, V>::DR;
    constexpr BlkF B = blk_fwd(K, sizeof(T), WRITE_O);
    constexpr int RM = ScanCfg<T, K, V>::read_mode(WRITE_O);
    constexpr int ES = sizeof(T), NI = B.SIZE / 1024;
    __shared__ __attribute__((aligned(16))) char lds[2][B.SIZE];

    const int h = blockIdx.x, n = blockIdx.y;
    const int vt = threadIdx.x >> 6;                      // this wave's column block; also its index for the shares
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    PHASE_CLOCK(p, (blockIdx.y * gridDim.x + blockIdx.x) * NW + vt, 0);

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
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const char* blocks = reinterpret_cast<const char*>(p.ws.W);

    struct Stage {
        Share<NI, NW> sh;
        Frag<T> ut[2], vtt;
    };
    auto load_share = [&](Stage& st, int cid) __attribute__((always_inline)) {
        st.sh.load(blocks + (chw0 + cid) * B.SIZE, vt);
    };
    auto load_own = [&](Stage& st, int cid) __attribute__((always_inline)) {
        if (!ScanCfg<T, K, V>::RING_OWN) return;
        const int64_t chw = chw0 + cid;
        ld_pair(p.ws.UT + (chw * VT + vt) * PAIR, st.ut[0], st.ut[1]);
        st.vtt = ld_tile(p.ws.VTT + (chw * VT + vt) * TILE);
    };
    auto load_stage = [&](Stage& st, int cid) __attribute__((always_inline)) {
        load_share(st, cid);
        load_own(st, cid);
    };

    // one chunk, shared operands from the LDS slot, own operands in registers
    auto step = [&](const char* slot, Frag<T> ut0, Frag<T> ut1, Frag<T> vtt, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + cid;
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        const T* sW = reinterpret_cast<const T*>(slot + B.W);
        const T* sBGT = reinterpret_cast<const T*>(slot + B.BGT);
        const T* sKGT = reinterpret_cast<const T*>(slot + B.KGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + B.EGL);
        if (!ScanCfg<T, K, V>::RING_OWN) {
            ld_pair(p.ws.UT + (chw * VT + vt) * PAIR, ut0, ut1);
            vtt = ld_tile(p.ws.VTT + (chw * VT + vt) * TILE);
        }
        // All LDS reads of the step are issued up front, in the order of use: left to itself the compiler sinks
        // each read to just before its product and the step pays the LDS latency half a dozen times over.
        Frag<T> w[2][KT], qg[WRITE_O ? KT : 1], aqk, aqb[2], kgt[KT], bgt[2][KT];
        f32x4 egl[KT];
        auto read_w = [&](int kp) __attribute__((always_inline)) {
            ld_pair(sW + (0 * KT2 + kp) * PAIR, w[0][2 * kp], w[0][2 * kp + 1]);
            ld_pair(sW + (1 * KT2 + kp) * PAIR, w[1][2 * kp], w[1][2 * kp + 1]);
        };
        auto read_qg = [&](int kp) __attribute__((always_inline)) {
            ld_pair(reinterpret_cast<const T*>(slot + B.QG) + kp * PAIR, qg[2 * kp], qg[2 * kp + 1]);
        };
        auto read_upd = [&](int kp) __attribute__((always_inline)) {
            ld_pair(sKGT + kp * PAIR, kgt[2 * kp], kgt[2 * kp + 1]);
            ld_pair(sBGT + (0 * KT2 + kp) * PAIR, bgt[0][2 * kp], bgt[0][2 * kp + 1]);
            ld_pair(sBGT + (1 * KT2 + kp) * PAIR, bgt[1][2 * kp], bgt[1][2 * kp + 1]);
            egl[2 * kp] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp) + 4 * g);
            egl[2 * kp + 1] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp + 1) + 4 * g);
        };
        if (RM) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_w(kp);
            if (WRITE_O) {
#pragma unroll
                for (int kp = 0; kp < KT2; ++kp) read_qg(kp);
            }
        }
        if (WRITE_O) {
            ld_pair(reinterpret_cast<const T*>(slot + B.AQB), aqb[0], aqb[1]);
            aqk = ld_tile(reinterpret_cast<const T*>(slot + B.AQK));
        }
        if (RM == 2) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
        }
        if (RM) __builtin_amdgcn_sched_barrier(0);
        Frag<T> sb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sb[kt] = to_frag<T>(S[kt]);
        // v_new^T (rows value, inner token) = u^T + S^T w^T
        f32x4 vn[2] = {to_f32(ut0), to_f32(ut1)};
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!RM) read_w(kp);
            vn[0] = mm2s<0>(sb[2 * kp], w[0][2 * kp], sb[2 * kp + 1], w[0][2 * kp + 1], vn[0]);
            vn[1] = mm2s<0>(sb[2 * kp], w[1][2 * kp], sb[2 * kp + 1], w[1][2 * kp + 1], vn[1]);
        }
        if (RM == 1) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
            __builtin_amdgcn_sched_barrier(0);
        }
        const Frag<T> vnb[2] = {to_frag<T>(vn[0]), to_frag<T>(vn[1])};
        if (!WRITE_O) {
            // checkpoint of the entering state and v_new, as the fragments held here (tile pairs, 16 bytes per
            // lane, whole cache lines): the chunk_grad kernel turns them the way it needs them
            T* hc = p.ws.HC + chw * (K * V) + vt * PAIR;
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) st_pair2(hc + kp * VT * PAIR, sb[2 * kp], sb[2 * kp + 1]);
            st_pair2(p.ws.VN + chw * (2 * CH * V) + vt * PAIR, vnb[0], vnb[1]);
        }
        if (WRITE_O) {
            // o (rows token, inner value) = qg S + A_qk v + sum_s A_qb^s v_new_s
            f32x4 o = zero4();
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) {
                if (!RM) read_qg(kp);
                o = mm2s<1>(qg[2 * kp], sb[2 * kp], qg[2 * kp + 1], sb[2 * kp + 1], o);
            }
            o = mm(aqk, vtt, o);
            o = mm2s<2>(aqb[0], vnb[0], aqb[1], vnb[1], o);
            if (c < len) st_frag(p.o + ((tok0 + c) * H + h) * V + 16 * vt + 4 * g, to_frag<T>(o));
        }
        // S <- exp(g_last) S + kg^T v + sum_s bg_s^T v_new_s
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!RM) read_upd(kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                f32x4 x = S[kt] * egl[kt];
                x = mm(vtt, kgt[kt], x);
                x = mm2s<3>(vnb[0], bgt[0][kt], vnb[1], bgt[1][kt], x);
                S[kt] = x;
            }
        }
    };

#ifdef HDLA_PHASE_TIMING
    long long tacc[3] = {0, 0, 0}, tlast = clock64();
#define TCK(i) do { long long t_ = clock64(); tacc[((i) + 2) % 3] += t_ - tlast; tlast = t_; } while (0)
#else
#define TCK(i) do { } while (0)
#endif
    const int nchunks = c1 - c0;
    if (nchunks > 0) {
        // Every global load of the main loop is unconditional (prefetch indices are clamped to the last chunk): a
        // load that may or may not have been issued would make the compiler wait for all outstanding loads.
        Stage ring[DR];
#pragma unroll
        for (int d = 0; d < DR; ++d) load_stage(ring[d], min(c0 + d, c1 - 1));
        ring[0].sh.to_lds(lds[0], vt);
        const int nfull = nchunks / DR;
#pragma unroll 1
        for (int gi = 0; gi < nfull; ++gi) {
            const int base = c0 + gi * DR;
#pragma unroll
            for (int j = 0; j < DR; ++j) {                 // DR is even: chunk base+j lives in LDS slot j & 1
                const int cid = base + j;
                TCK(0);
                lds_barrier();                             // block of this chunk complete; other slot free again
                TCK(1);
                ring[(j + 1) % DR].sh.to_lds(lds[(j + 1) & 1], vt);                 // hand over the next chunk
                TCK(2);
                const int nxt = min(cid + DR, c1 - 1);
                load_share(ring[j], nxt);                  // this share went to LDS a step ago: refill it now
                step(lds[j & 1], ring[j].ut[0], ring[j].ut[1], ring[j].vtt, cid);
                // the own tiles are refilled only after their last use: a register that is loaded while its old
                // value is still live needs a copy, and the copy would wait for the load just issued
                load_own(ring[j], nxt);
            }
        }
#pragma unroll 1
        for (int cid = c0 + nfull * DR; cid < c1; ++cid) {  // fewer than DR chunks left: one at a time
            Stage st;
            load_stage(st, cid);
            lds_barrier();
            st.sh.to_lds(lds[0], vt);
            lds_barrier();
            step(lds[0], st.ut[0], st.ut[1], st.vtt, cid);
        }
    }
    PHASE_CLOCK(p, (blockIdx.y * gridDim.x + blockIdx.x) * NW + vt, 1);
#ifdef HDLA_PHASE_TIMING
    {
        const int blk_ = (blockIdx.y * gridDim.x + blockIdx.x) * NW + vt;
        if (p.phase_clk && blk_ < 64 && lane_id() == 0)
            for (int i = 0; i < 3; ++i) p.phase_clk[blk_ * 16 + 8 + i] = tacc[i];
    }
#endif
    if (p.ht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
template <typename T, int K, int V>
__global__ __launch_bounds__(V * 4) void scan_bwd_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NW = ScanCfg<T, K, V>::NW, DR = ScanCfg<T, K, V>::DR;
    constexpr BlkB B = blk_bwd(K, sizeof(T));
    constexpr int RM = ScanCfg<T, K, V>::read_mode(false);
    constexpr int NI = B.SIZE / 1024;
    __shared__ __attribute__((aligned(16))) char lds[2][B.SIZE];

    const int h = blockIdx.x, n = blockIdx.y;
    const int vt = threadIdx.x >> 6;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    PHASE_CLOCK(p, (blockIdx.y * gridDim.x + blockIdx.x) * NW + vt, 0);

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
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const char* blocks = reinterpret_cast<const char*>(p.ws.BG);

    struct Stage {
        Share<NI, NW> sh;
        Frag<T> don;      // rows past the end of a ragged chunk alias its last row and are zeroed where used
    };
    auto load_share = [&](Stage& st, int cid) __attribute__((always_inline)) {
        st.sh.load(blocks + (chw0 + cid) * B.SIZE, vt);
    };
    auto load_own = [&](Stage& st, int cid) __attribute__((always_inline)) {
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        st.don = ld_frag(p.dout + ((tok0 + min(c, len - 1)) * H + h) * V + 16 * vt + 4 * g);
    };
    auto load_stage = [&](Stage& st, int cid) __attribute__((always_inline)) {
        load_share(st, cid);
        load_own(st, cid);
    };

    auto step = [&](const char* slot, Frag<T> don, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + cid;
        const T* sBG = reinterpret_cast<const T*>(slot + B.BG);
        const T* sWT = reinterpret_cast<const T*>(slot + B.WT);
        const T* sQGT = reinterpret_cast<const T*>(slot + B.QGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + B.EGL);
        // all LDS reads first, in the order of use (see the forward scan)
        Frag<T> aq[2], bg[2][KT], qgt[KT], wt[2][KT];
        f32x4 egl[KT];
        auto read_bg = [&](int kp) __attribute__((always_inline)) {
            ld_pair(sBG + (0 * KT2 + kp) * PAIR, bg[0][2 * kp], bg[0][2 * kp + 1]);
            ld_pair(sBG + (1 * KT2 + kp) * PAIR, bg[1][2 * kp], bg[1][2 * kp + 1]);
        };
        auto read_upd = [&](int kp) __attribute__((always_inline)) {
            ld_pair(sQGT + kp * PAIR, qgt[2 * kp], qgt[2 * kp + 1]);
            ld_pair(sWT + (0 * KT2 + kp) * PAIR, wt[0][2 * kp], wt[0][2 * kp + 1]);
            ld_pair(sWT + (1 * KT2 + kp) * PAIR, wt[1][2 * kp], wt[1][2 * kp + 1]);
            egl[2 * kp] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp) + 4 * g);
            egl[2 * kp + 1] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp + 1) + 4 * g);
        };
        ld_pair(reinterpret_cast<const T*>(slot + B.AQBT), aq[0], aq[1]);
        if (RM) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_bg(kp);
        }
        if (RM == 2) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
        }
        if (RM) __builtin_amdgcn_sched_barrier(0);
        Frag<T> dsb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) dsb[kt] = to_frag<T>(dS[kt]);
        const int len = (int)min((int64_t)CH, eos - (bos + (int64_t)(cid - c0) * CH));
        if (c >= len) don = zero_frag<T>();
        const Frag<T> doT = transpose(don, ident);          // rows value, inner token
        // dv_new_s^T (rows value, inner token) = do^T A_qb^s + dS^T bg_s^T
        f32x4 dvn[2];
        dvn[0] = mm(doT, aq[0], zero4());
        dvn[1] = mm(doT, aq[1], zero4());
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!RM) read_bg(kp);
            dvn[0] = mm2s<4>(dsb[2 * kp], bg[0][2 * kp], dsb[2 * kp + 1], bg[0][2 * kp + 1], dvn[0]);
            dvn[1] = mm2s<4>(dsb[2 * kp], bg[1][2 * kp], dsb[2 * kp + 1], bg[1][2 * kp + 1], dvn[1]);
        }
        if (RM == 1) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
            __builtin_amdgcn_sched_barrier(0);
        }
        const Frag<T> dvb[2] = {to_frag<T>(dvn[0]), to_frag<T>(dvn[1])};
        // gradient of the state leaving the chunk and of v_new, as the fragments held here (tile pairs)
        T* dhc = p.ws.DHC + chw * (K * V) + vt * PAIR;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) st_pair2(dhc + kp * VT * PAIR, dsb[2 * kp], dsb[2 * kp + 1]);
        st_pair2(p.ws.DVN + chw * (2 * CH * V) + vt * PAIR, dvb[0], dvb[1]);
        // dS <- exp(g_last) dS + qg^T do + sum_s w_s^T dv_new_s
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!RM) read_upd(kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                f32x4 x = dS[kt] * egl[kt];
                x = mm(doT, qgt[kt], x);
                x = mm2s<5>(dvb[0], wt[0][kt], dvb[1], wt[1][kt], x);
                dS[kt] = x;
            }
        }
    };

    const int nchunks = c1 - c0;
    if (nchunks > 0) {
        Stage ring[DR];
#pragma unroll
        for (int d = 0; d < DR; ++d) load_stage(ring[d], max(c1 - 1 - d, c0));
        ring[0].sh.to_lds(lds[0], vt);
        const int nfull = nchunks / DR;
#pragma unroll 1
        for (int gi = 0; gi < nfull; ++gi) {
            const int base = c1 - 1 - gi * DR;
#pragma unroll
            for (int j = 0; j < DR; ++j) {
                const int cid = base - j;
                lds_barrier();
                ring[(j + 1) % DR].sh.to_lds(lds[(j + 1) & 1], vt);
                const int nxt = max(cid - DR, c0);
                load_share(ring[j], nxt);
                step(lds[j & 1], ring[j].don, cid);
                load_own(ring[j], nxt);                    // after the last use of the old value: no copy, no wait
            }
        }
#pragma unroll 1
        for (int cid = c1 - 1 - nfull * DR; cid >= c0; --cid) {
            Stage st;
            load_stage(st, cid);
            lds_barrier();
            st.sh.to_lds(lds[0], vt);
            lds_barrier();
            step(lds[0], st.don, cid);
        }
    }
    PHASE_CLOCK(p, (blockIdx.y * gridDim.x + blockIdx.x) * NW + vt, 1);
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
    dim3 grid(a.H, a.st.N), block(V * 4);
    if (write_o) hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}
template <typename T, int K, int V>
static hipError_t launch_scan_bwd_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.H, a.st.N), block(V * 4);
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
