// The two inter-chunk state scans: the only sequential part of the chunked operator.
//
// scan_fwd replaces HRDPLR/fwd_triton.py:808-968 (state recurrence, h checkpoints, v_new, final state) and, in
// the forward pass, also HRDPLR/fwd_triton.py:984-1095 (the output o), so the forward pass never writes h.
// scan_bwd replaces HRDPLR/bwd_triton.py:127-222 (reverse recurrence of the state gradient, dh checkpoints,
// dh0) fused with the dv_new part of HRDPLR/bwd_triton.py:30-105.
//
// One workgroup per (sequence, head), one wavefront per 16-column block of the fp32 state.  A wave keeps its
// K x 16 block in registers as the row fragment of S^T (rows = value column, inner = channel), which is at once
// the operand layout of the next product: w S, qg S and the rank updates chain through registers with no
// cross-lane movement.
//
// What bounds a step is not arithmetic but operand delivery: a wave may have at most 63 memory instructions in
// flight, and every wave of a head needs the same w / kg / bg / qg tiles.  So the waves of a workgroup split the
// chunk's shared operand block (one contiguous block per chunk, written by the prep kernel) between them:
// each wave fetches its share of the blocks of the next few chunks into registers (16 bytes per lane, a few
// instructions per chunk) and hands them to LDS two chunks ahead of their use; all waves read their operands
// from LDS.  Three LDS slots rotate, with ONE LDS-only barrier per chunk (global loads stay in flight across it):
//
//   step t:  barrier                      block t+1 (written during step t-1) becomes visible
//            share of block t+2 -> slot (t+2) % 3          (its last readers finished before the barrier)
//            read the operands of the state update of chunk t from slot t % 3
//            phase 1: v_new (operands already in registers, read during step t-1)
//            read the phase-1 operands of chunk t+1 from slot (t+1) % 3
//            phase 2: state update
//
// so every LDS read has a phase of matrix products between its issue and its first use.
//
// Stores go through LDS as well, to waves that do nothing else ("store waves").  Memory instructions of one wave
// complete in order, and the acknowledgement of a store takes several times as long as a load takes to return
// (much longer still right after a kernel that left the L2 full of dirty lines, as the prep kernel does): a wave
// that both stores its results and waits for prefetched operands ends up waiting for its own stores.  The
// computing waves therefore leave a chunk's results in an LDS outbox laid out like the chunk's record in global
// memory, and the store waves copy the outbox of the previous chunk out while the next chunk is computed; they
// never wait for anything but the per-chunk barrier.
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

constexpr int NSLOT = 3;

template <typename T, int K, int V> struct ScanCfg {
    static constexpr int NW = V / 16;                 // computing wavefronts per workgroup
    static constexpr int KB = K * (int)sizeof(T);     // bytes of one operand row
    // Store waves.  Only where eight waves leave every computing wave the registers it needs: not at V = 128
    // (eight computing waves already) and not for operand rows beyond 128 bytes.
    static constexpr int NH = (V == 64 && KB <= 128) ? 4 : 0;
    static constexpr int THREADS = 64 * (NW + NH);
    // Depth of the register ring of block shares and own tiles (chunks in flight from global memory); a multiple
    // of the number of slots so that slot numbers are static in the unrolled loop; 0: no ring, one chunk at a time.
    static constexpr int DR = KB <= 128 ? 6 : KB <= 256 ? 3 : 0;
    // Whether LDS reads are issued a phase ahead of their use as described above, or left where the compiler
    // puts them (the shapes whose operands would not fit the register file twice over).
    static constexpr bool pipelined(bool with_o) { return KB <= 128 || (KB <= 256 && !(V == 128 && with_o)); }
    // ... and whether that includes the operands of the state update (80 registers at KB = 256, too many for the
    // eight-wave workgroups of V = 128, which have 256 registers per lane)
    static constexpr bool early_update_reads() { return KB <= 128 || (KB <= 256 && V == 64); }
};

// one wave's share of a shared operand block: the 1-KiB pieces w, w+NW, ... of its NI pieces
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

// One store wave's part of copying an outbox record of NP 1-KiB pieces to global memory; piece i goes to dst(i).
template <int NP, int NH, typename Dst>
__device__ __forceinline__ void copy_out(const char* outbox, int hw, Dst dst) {
    const int l = lane_id();
#pragma unroll
    for (int j = 0; j < (NP + NH - 1) / NH; ++j) {
        const int i = hw + j * NH;
        if (i < NP) *reinterpret_cast<i32x4*>(dst(i) + l * 16) = *reinterpret_cast<const i32x4*>(outbox + i * 1024 + l * 16);
    }
}

// ---- forward -------------------------------------------------------------------------------------------------
// LDS of the forward scan: the three operand slots, then (with store waves) two outboxes.  Backward pass: an
// outbox is the chunk's checkpoint record, [K/32][V/16] tile pairs of the state then [V/16] tile pairs of v_new,
// exactly as in global memory.  Forward pass: the 16 x V output rows, padded by 16 bytes a row against bank
// conflicts.
template <typename T, int K, int V, bool WRITE_O> struct FwdLds {
    static constexpr int ES = sizeof(T), NH = ScanCfg<T, K, V>::NH;
    static constexpr int SLOT = blk_fwd(K, ES, WRITE_O).SIZE;
    static constexpr int OROW = V * ES + 16;
    static constexpr int OB_HC = K * V * ES, OB = WRITE_O ? CH * OROW : OB_HC + 2 * CH * V * ES;
    static constexpr int BYTES = NSLOT * SLOT + (NH ? 2 * OB : 0);
};

template <typename T, int K, int V, bool WRITE_O>
__device__ __forceinline__ void scan_fwd_body(const ChunkArgs<T>& p, char* smem) {
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NW = ScanCfg<T, K, V>::NW, DR = ScanCfg<T, K, V>::DR;
    constexpr int NH = ScanCfg<T, K, V>::NH, ES = sizeof(T);
    constexpr BlkF B = blk_fwd(K, sizeof(T), WRITE_O);
    constexpr bool PIPE = ScanCfg<T, K, V>::pipelined(WRITE_O);
    constexpr bool PIPE_UPD = PIPE && ScanCfg<T, K, V>::early_update_reads();
    constexpr int NI = B.SIZE / 1024;
    typedef FwdLds<T, K, V, WRITE_O> L;
    constexpr int OROW = L::OROW, OB_HC = L::OB_HC, OB = L::OB;
    char (*lds)[B.SIZE] = reinterpret_cast<char (*)[B.SIZE]>(smem);
    char (*outbox)[OB] = reinterpret_cast<char (*)[OB]>(smem + NSLOT * B.SIZE);

    const int h = blockIdx.x, n = blockIdx.y;
    const int vt = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // column block of a computing wave
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const int nchunks = c1 - c0;

    if (NH && vt >= NW) {
        // ---- store wave: one barrier for the computing waves' prologue, one per chunk, one to close; after the
        // barrier of step t the outbox of chunk t-1 is complete, and it is overwritten only after the barrier of t+1
        if (nchunks <= 0) return;
        const int hw = vt - NW;
        lds_barrier();
        for (int t = 0; t <= nchunks; ++t) {
            lds_barrier();
            if (t == 0) continue;
            const int cid = c0 + t - 1;
            const char* ob = outbox[(t - 1) & 1];
            if (WRITE_O) {
                // rows of o: 16-byte pieces, LPR lanes a row
                constexpr int LPR = V * ES / 16, RPI = 64 / LPR;
                const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
                const int len = (int)min((int64_t)CH, eos - tok0);
#pragma unroll
                for (int r0 = hw * RPI; r0 < CH; r0 += (NH ? NH : 1) * RPI) {
                    const int r = r0 + l / LPR, e = (l % LPR) * 16;
                    if (r < len)
                        *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(p.o + ((tok0 + r) * H + h) * V) + e) =
                            *reinterpret_cast<const i32x4*>(ob + r * OROW + e);
                }
            } else {
                char* hc = reinterpret_cast<char*>(p.ws.HC + (chw0 + cid) * (K * V));
                char* vn = reinterpret_cast<char*>(p.ws.VN + (chw0 + cid) * (2 * CH * V));
                copy_out<OB / 1024, NH ? NH : 1>(ob, hw, [&](int i) { return i < OB_HC / 1024 ? hc + i * 1024 : vn + (i - OB_HC / 1024) * 1024; });
            }
        }
        return;
    }

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
    const int last = c1 - 1;
    // block of chunk cid; indices past the end of the sequence are clamped, so every load is unconditional (a load
    // that may or may not have been issued would make the compiler wait for all outstanding loads)
    auto blk = [&](int cid) __attribute__((always_inline)) {
        return reinterpret_cast<const char*>(p.ws.W) + (chw0 + min(cid, last)) * B.SIZE;
    };
    struct Own { Frag<T> ut[2], vtt; };                   // the tiles only this wave reads
    auto load_own = [&](Own& o, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + min(cid, last);
        ld_pair(p.ws.UT + (chw * VT + vt) * PAIR, o.ut[0], o.ut[1]);
        o.vtt = ld_tile(p.ws.VTT + (chw * VT + vt) * TILE);
    };

    Frag<T> w[2][KT];                                     // phase-1 operands; when pipelined, read a step ahead
    auto read_w = [&](const char* slot, int kp) __attribute__((always_inline)) {
        const T* sW = reinterpret_cast<const T*>(slot + B.W);
        ld_pair(sW + (0 * KT2 + kp) * PAIR, w[0][2 * kp], w[0][2 * kp + 1]);
        ld_pair(sW + (1 * KT2 + kp) * PAIR, w[1][2 * kp], w[1][2 * kp + 1]);
    };
    auto read_w_all = [&](const char* slot) __attribute__((always_inline)) {
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) read_w(slot, kp);
    };

    // one chunk: shared operands from `slot`, the phase-1 operands of the next chunk from `slot_next`, results
    // that go to global memory into the outbox `ob` (when there are store waves)
    auto step = [&](const char* slot, const char* slot_next, char* ob, Own own, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + cid;
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        const T* sBGT = reinterpret_cast<const T*>(slot + B.BGT);
        const T* sKGT = reinterpret_cast<const T*>(slot + B.KGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + B.EGL);
        Frag<T> qg[WRITE_O ? KT : 1], aqk, aqb[2], kgt[KT], bgt[2][KT];
        f32x4 egl[KT];
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
        if (WRITE_O) {
            if (PIPE) {
#pragma unroll
                for (int kp = 0; kp < KT2; ++kp) read_qg(kp);
            }
            ld_pair(reinterpret_cast<const T*>(slot + B.AQB), aqb[0], aqb[1]);
            aqk = ld_tile(reinterpret_cast<const T*>(slot + B.AQK));
        }
        if (PIPE_UPD) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
        }
        if (PIPE) __builtin_amdgcn_sched_barrier(0);      // the reads above stay above the products below
        Frag<T> sb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sb[kt] = to_frag<T>(S[kt]);
        // v_new^T (rows value, inner token) = u^T + S^T w^T
        f32x4 vn[2] = {to_f32(own.ut[0]), to_f32(own.ut[1])};
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!PIPE) read_w(slot, kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                vn[0] = mm(sb[kt], w[0][kt], vn[0]);
                vn[1] = mm(sb[kt], w[1][kt], vn[1]);
            }
        }
        f32x4 o = zero4();
        if (WRITE_O) {
            // o (rows token, inner value) = qg S + A_qk v + sum_s A_qb^s v_new_s; the first two terms here
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) {
                if (!PIPE) read_qg(kp);
                o = mm(qg[2 * kp], sb[2 * kp], o);
                o = mm(qg[2 * kp + 1], sb[2 * kp + 1], o);
            }
            o = mm(aqk, own.vtt, o);
        }
        if (PIPE) {
            __builtin_amdgcn_sched_barrier(0);
            read_w_all(slot_next);                        // the products above have taken their operands already
            __builtin_amdgcn_sched_barrier(0);
        }
        const Frag<T> vnb[2] = {to_frag<T>(vn[0]), to_frag<T>(vn[1])};
        if (!WRITE_O) {
            // checkpoint of the entering state and v_new, as the fragments held here (tile pairs, 16 bytes per
            // lane, whole cache lines): the chunk_grad kernel turns them the way it needs them
            T* hc = (NH ? reinterpret_cast<T*>(ob) : p.ws.HC + chw * (K * V)) + vt * PAIR;
            T* vnp = (NH ? reinterpret_cast<T*>(ob + OB_HC) : p.ws.VN + chw * (2 * CH * V)) + vt * PAIR;
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) st_pair2(hc + kp * VT * PAIR, sb[2 * kp], sb[2 * kp + 1]);
            st_pair2(vnp, vnb[0], vnb[1]);
        }
        if (WRITE_O) {
            o = mm(aqb[0], vnb[0], o);
            o = mm(aqb[1], vnb[1], o);
            if (NH) st_frag(reinterpret_cast<T*>(ob + c * OROW) + 16 * vt + 4 * g, to_frag<T>(o));
            else if (c < len) st_frag(p.o + ((tok0 + c) * H + h) * V + 16 * vt + 4 * g, to_frag<T>(o));
        }
        // S <- exp(g_last) S + kg^T v + sum_s bg_s^T v_new_s
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!PIPE_UPD) read_upd(kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                f32x4 x = S[kt] * egl[kt];
                x = mm(own.vtt, kgt[kt], x);
                x = mm(vnb[0], bgt[0][kt], x);
                x = mm(vnb[1], bgt[1][kt], x);
                S[kt] = x;
            }
        }
    };

    if (nchunks > 0) {
        int done = 0;
        if constexpr (DR > 0) {
            Share<NI, NW> sh[DR];
            Own own[DR];
#pragma unroll
            for (int d = 0; d < DR; ++d) {
                sh[d].load(blk(c0 + d), vt);
                load_own(own[d], c0 + d);
            }
            sh[0].to_lds(lds[0], vt);
            sh[1].to_lds(lds[1], vt);
            sh[0].load(blk(c0 + DR), vt);
            sh[1].load(blk(c0 + DR + 1), vt);
            lds_barrier();
            if (PIPE) read_w_all(lds[0]);
            const int nfull = nchunks / DR;
#pragma unroll 1
            for (int gi = 0; gi < nfull; ++gi) {
                const int base = c0 + gi * DR;
#pragma unroll
                for (int j = 0; j < DR; ++j) {             // DR is a multiple of NSLOT: chunk base+j lives in slot j % 3
                    const int cid = base + j;
                    lds_barrier();
#ifdef HDLA_PHASE_TIMING
                    if (!WRITE_O && p.phase_clk && blockIdx.x == 3 && blockIdx.y == 1 && threadIdx.x == 0 && cid - c0 < 1000) p.phase_clk[cid - c0] = wall_clock64();
#endif
                    sh[(j + 2) % DR].to_lds(lds[(j + 2) % NSLOT], vt);
                    sh[(j + 2) % DR].load(blk(cid + 2 + DR), vt);
                    step(lds[j % NSLOT], lds[(j + 1) % NSLOT], outbox[(cid - c0) & 1], own[j], cid);
                    // refilled only after the last use: a register that is loaded while its old value is still
                    // live needs a copy, and the copy would wait for the load just issued
                    load_own(own[j], cid + DR);
                }
            }
            done = nfull * DR;
        } else {
            Share<NI, NW> tmp;
            tmp.load(blk(c0), vt);
            tmp.to_lds(lds[0], vt);
            tmp.load(blk(c0 + 1), vt);
            tmp.to_lds(lds[1], vt);
            lds_barrier();
            if (PIPE) read_w_all(lds[0]);
        }
        // what is left (fewer than DR chunks, or all of them without a ring): one chunk at a time, same protocol
        if (done < nchunks) {
            Own cur;
            load_own(cur, c0 + done);
#pragma unroll 1
            for (int t = done; t < nchunks; ++t) {
                const int cid = c0 + t;
                lds_barrier();
                Share<NI, NW> tmp;
                tmp.load(blk(cid + 2), vt);
                Own nxt;
                load_own(nxt, cid + 1);
                step(lds[t % NSLOT], lds[(t + 1) % NSLOT], outbox[t & 1], cur, cid);
                tmp.to_lds(lds[(t + 2) % NSLOT], vt);
                cur = nxt;
            }
        }
        if (NH) lds_barrier();                            // hands the last outbox to the store waves
    }
    if (p.ht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
// LDS of the reverse scan: three operand slots, then two outboxes holding the chunk's record of dS ([K/32][V/16]
// tile pairs) then dv_new ([V/16] tile pairs), as in global memory.
template <typename T, int K, int V> struct BwdLds {
    static constexpr int ES = sizeof(T), NH = ScanCfg<T, K, V>::NH;
    static constexpr int SLOT = blk_bwd(K, ES).SIZE;
    static constexpr int OB_HC = K * V * ES, OB = OB_HC + 2 * CH * V * ES;
    static constexpr int BYTES = NSLOT * SLOT + (NH ? 2 * OB : 0);
};

template <typename T, int K, int V>
__device__ __forceinline__ void scan_bwd_body(const ChunkArgs<T>& p, char* smem) {
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NW = ScanCfg<T, K, V>::NW, DR = ScanCfg<T, K, V>::DR;
    constexpr int NH = ScanCfg<T, K, V>::NH, ES = sizeof(T);
    constexpr BlkB B = blk_bwd(K, sizeof(T));
    constexpr bool PIPE = ScanCfg<T, K, V>::pipelined(false);
    constexpr bool PIPE_UPD = PIPE && ScanCfg<T, K, V>::early_update_reads();
    constexpr int NI = B.SIZE / 1024;
    typedef BwdLds<T, K, V> L;
    constexpr int OB_HC = L::OB_HC, OB = L::OB;
    char (*lds)[B.SIZE] = reinterpret_cast<char (*)[B.SIZE]>(smem);
    char (*outbox)[OB] = reinterpret_cast<char (*)[OB]>(smem + NSLOT * B.SIZE);

    const int h = blockIdx.x, n = blockIdx.y;
    const int vt = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const int nchunks = c1 - c0;

    if (NH && vt >= NW) {
        // ---- store wave (see the forward scan); step t handles chunk c1-1-t
        if (nchunks <= 0) return;
        const int hw = vt - NW;
        lds_barrier();
        for (int t = 0; t <= nchunks; ++t) {
            lds_barrier();
            if (t == 0) continue;
            const int cid = c1 - t;
            char* hc = reinterpret_cast<char*>(p.ws.DHC + (chw0 + cid) * (K * V));
            char* vn = reinterpret_cast<char*>(p.ws.DVN + (chw0 + cid) * (2 * CH * V));
            copy_out<OB / 1024, NH ? NH : 1>(outbox[(t - 1) & 1], hw,
                                              [&](int i) { return i < OB_HC / 1024 ? hc + i * 1024 : vn + (i - OB_HC / 1024) * 1024; });
        }
        return;
    }

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
    // the scan runs from the last chunk to the first: step t handles chunk c1-1-t; indices before c0 are clamped
    auto blk = [&](int cid) __attribute__((always_inline)) {
        return reinterpret_cast<const char*>(p.ws.BG) + (chw0 + max(cid, c0)) * B.SIZE;
    };
    // rows of do; rows past the end of a ragged chunk alias its last row and are zeroed where used
    auto load_own = [&](Frag<T>& don, int cid) __attribute__((always_inline)) {
        const int64_t tok0 = bos + (int64_t)(max(cid, c0) - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        don = ld_frag(p.dout + ((tok0 + min(c, len - 1)) * H + h) * V + 16 * vt + 4 * g);
    };

    Frag<T> aq[2], bg[2][KT];                             // phase-1 operands; when pipelined, read a step ahead
    auto read_bg = [&](const char* slot, int kp) __attribute__((always_inline)) {
        const T* sBG = reinterpret_cast<const T*>(slot + B.BG);
        ld_pair(sBG + (0 * KT2 + kp) * PAIR, bg[0][2 * kp], bg[0][2 * kp + 1]);
        ld_pair(sBG + (1 * KT2 + kp) * PAIR, bg[1][2 * kp], bg[1][2 * kp + 1]);
    };
    auto read_p1_all = [&](const char* slot) __attribute__((always_inline)) {
        ld_pair(reinterpret_cast<const T*>(slot + B.AQBT), aq[0], aq[1]);
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) read_bg(slot, kp);
    };

    auto step = [&](const char* slot, const char* slot_next, char* ob, Frag<T> don, int cid) __attribute__((always_inline)) {
        const int64_t chw = chw0 + cid;
        const T* sWT = reinterpret_cast<const T*>(slot + B.WT);
        const T* sQGT = reinterpret_cast<const T*>(slot + B.QGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + B.EGL);
        Frag<T> qgt[KT], wt[2][KT];
        f32x4 egl[KT];
        auto read_upd = [&](int kp) __attribute__((always_inline)) {
            ld_pair(sQGT + kp * PAIR, qgt[2 * kp], qgt[2 * kp + 1]);
            ld_pair(sWT + (0 * KT2 + kp) * PAIR, wt[0][2 * kp], wt[0][2 * kp + 1]);
            ld_pair(sWT + (1 * KT2 + kp) * PAIR, wt[1][2 * kp], wt[1][2 * kp + 1]);
            egl[2 * kp] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp) + 4 * g);
            egl[2 * kp + 1] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp + 1) + 4 * g);
        };
        if (PIPE_UPD) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) read_upd(kp);
        }
        if (PIPE) __builtin_amdgcn_sched_barrier(0);
        else ld_pair(reinterpret_cast<const T*>(slot + B.AQBT), aq[0], aq[1]);
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
            if (!PIPE) read_bg(slot, kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                dvn[0] = mm(dsb[kt], bg[0][kt], dvn[0]);
                dvn[1] = mm(dsb[kt], bg[1][kt], dvn[1]);
            }
        }
        if (PIPE) {
            __builtin_amdgcn_sched_barrier(0);
            read_p1_all(slot_next);
            __builtin_amdgcn_sched_barrier(0);
        }
        const Frag<T> dvb[2] = {to_frag<T>(dvn[0]), to_frag<T>(dvn[1])};
        // gradient of the state leaving the chunk and of v_new, as the fragments held here (tile pairs)
        T* dhc = (NH ? reinterpret_cast<T*>(ob) : p.ws.DHC + chw * (K * V)) + vt * PAIR;
        T* dvp = (NH ? reinterpret_cast<T*>(ob + OB_HC) : p.ws.DVN + chw * (2 * CH * V)) + vt * PAIR;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) st_pair2(dhc + kp * VT * PAIR, dsb[2 * kp], dsb[2 * kp + 1]);
        st_pair2(dvp, dvb[0], dvb[1]);
        // dS <- exp(g_last) dS + qg^T do + sum_s w_s^T dv_new_s
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            if (!PIPE_UPD) read_upd(kp);
#pragma unroll
            for (int kt = 2 * kp; kt < 2 * kp + 2; ++kt) {
                f32x4 x = dS[kt] * egl[kt];
                x = mm(doT, qgt[kt], x);
                x = mm(dvb[0], wt[0][kt], x);
                x = mm(dvb[1], wt[1][kt], x);
                dS[kt] = x;
            }
        }
    };

    if (nchunks > 0) {
        const int first = c1 - 1;
        int done = 0;
        if constexpr (DR > 0) {
            Share<NI, NW> sh[DR];
            Frag<T> own[DR];
#pragma unroll
            for (int d = 0; d < DR; ++d) {
                sh[d].load(blk(first - d), vt);
                load_own(own[d], first - d);
            }
            sh[0].to_lds(lds[0], vt);
            sh[1].to_lds(lds[1], vt);
            sh[0].load(blk(first - DR), vt);
            sh[1].load(blk(first - DR - 1), vt);
            lds_barrier();
            if (PIPE) read_p1_all(lds[0]);
            const int nfull = nchunks / DR;
#pragma unroll 1
            for (int gi = 0; gi < nfull; ++gi) {
                const int base = first - gi * DR;
#pragma unroll
                for (int j = 0; j < DR; ++j) {
                    const int cid = base - j;
                    lds_barrier();
                    sh[(j + 2) % DR].to_lds(lds[(j + 2) % NSLOT], vt);
                    sh[(j + 2) % DR].load(blk(cid - 2 - DR), vt);
                    step(lds[j % NSLOT], lds[(j + 1) % NSLOT], outbox[(first - cid) & 1], own[j], cid);
                    load_own(own[j], cid - DR);            // after the last use of the old value: no copy, no wait
                }
            }
            done = nfull * DR;
        } else {
            Share<NI, NW> tmp;
            tmp.load(blk(first), vt);
            tmp.to_lds(lds[0], vt);
            tmp.load(blk(first - 1), vt);
            tmp.to_lds(lds[1], vt);
            lds_barrier();
            if (PIPE) read_p1_all(lds[0]);
        }
        if (done < nchunks) {
            Frag<T> cur;
            load_own(cur, first - done);
#pragma unroll 1
            for (int t = done; t < nchunks; ++t) {
                const int cid = first - t;
                lds_barrier();
                Share<NI, NW> tmp;
                tmp.load(blk(cid - 2), vt);
                Frag<T> nxt;
                load_own(nxt, cid - 1);
                step(lds[t % NSLOT], lds[(t + 1) % NSLOT], outbox[t & 1], cur, cid);
                tmp.to_lds(lds[(t + 2) % NSLOT], vt);
                cur = nxt;
            }
        }
        if (NH) lds_barrier();
    }
    if (p.dh0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.dh0[soff + (int64_t)(16 * kt + 4 * g + i) * V] = dS[kt][i];
    }
}

// ---- kernels ---------------------------------------------------------------------------------------------------
template <typename T, int K, int V, bool WRITE_O>
__global__ __launch_bounds__((ScanCfg<T, K, V>::THREADS)) void scan_fwd_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[FwdLds<T, K, V, WRITE_O>::BYTES];
    scan_fwd_body<T, K, V, WRITE_O>(p, smem);
}
template <typename T, int K, int V>
__global__ __launch_bounds__((ScanCfg<T, K, V>::THREADS)) void scan_bwd_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[BwdLds<T, K, V>::BYTES];
    scan_bwd_body<T, K, V>(p, smem);
}
// Both scans of the backward pass in one launch: they depend on the prep kernel only, not on each other, and each
// occupies one workgroup per (sequence, head), a fraction of the machine.  blockIdx.z picks the direction.
template <typename T, int K, int V>
__global__ __launch_bounds__((ScanCfg<T, K, V>::THREADS)) void scan_pair_kernel(ChunkArgs<T> p) {
    constexpr int NF = FwdLds<T, K, V, false>::BYTES, NB = BwdLds<T, K, V>::BYTES;
    __shared__ __attribute__((aligned(16))) char smem[NF > NB ? NF : NB];
    if (blockIdx.z == 0) scan_fwd_body<T, K, V, false>(p, smem);
    else scan_bwd_body<T, K, V>(p, smem);
}

// ---- launchers -----------------------------------------------------------------------------------------------
template <typename T, int K, int V>
static hipError_t launch_scan_fwd_kv(const ChunkArgs<T>& a, bool write_o, hipStream_t stream) {
    dim3 grid(a.H, a.st.N), block(ScanCfg<T, K, V>::THREADS);
    if (write_o) hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}
template <typename T, int K, int V>
static hipError_t launch_scan_bwd_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.H, a.st.N), block(ScanCfg<T, K, V>::THREADS);
    hipLaunchKernelGGL((scan_bwd_kernel<T, K, V>), grid, block, 0, stream, a);
    return hipGetLastError();
}
template <typename T, int K, int V>
static hipError_t launch_scan_pair_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.H, a.st.N, 2), block(ScanCfg<T, K, V>::THREADS);
    hipLaunchKernelGGL((scan_pair_kernel<T, K, V>), grid, block, 0, stream, a);
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
template <typename T>
hipError_t launch_scan_pair(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_scan_pair_kv<T, 64, 64>(a, stream);
    if (K == 128 && V == 128) return launch_scan_pair_kv<T, 128, 128>(a, stream);
    if (K == 64 && V == 128) return launch_scan_pair_kv<T, 64, 128>(a, stream);
    if (K == 128 && V == 64) return launch_scan_pair_kv<T, 128, 64>(a, stream);
    return hipErrorInvalidValue;
}
template hipError_t launch_scan_fwd<bf16>(const ChunkArgs<bf16>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_fwd<float>(const ChunkArgs<float>&, int, int, bool, hipStream_t);
template hipError_t launch_scan_bwd<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_scan_bwd<float>(const ChunkArgs<float>&, int, int, hipStream_t);
template hipError_t launch_scan_pair<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_scan_pair<float>(const ChunkArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
