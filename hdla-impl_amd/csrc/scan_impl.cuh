// The two inter-chunk state scans: the only sequential part of the chunked operator.
//
// scan_fwd replaces HRDPLR/fwd_triton.py:808-968 (state recurrence, h checkpoints, v_new, final state) and, in
// the forward pass, also HRDPLR/fwd_triton.py:984-1095 (the output o), so the forward pass never writes h.
// scan_bwd replaces HRDPLR/bwd_triton.py:127-222 (reverse recurrence of the state gradient, dh checkpoints,
// dh0) fused with the dv_new part of HRDPLR/bwd_triton.py:30-105.
//
// A computing wave owns one 16-column block of the fp32 state of a (sequence, head) for the whole sequence, in
// registers as the row fragment of S^T (rows = value column, inner = channel), which is at once the operand
// layout of the next product: w S, qg S and the rank updates chain through registers with no cross-lane
// movement.  A workgroup holds NWC such waves; a head's V/16 column blocks are split over (V/16)/NWC workgroups.
//
// What bounds a step without the measures below is not arithmetic but memory: one compute unit sustains only a few
// tens of GB/s of loads that miss to HBM however many it has in flight, a wave may have at most 63 memory
// instructions outstanding and they complete in order, and all column blocks of a head need the same w / kg / bg /
// qg tiles.  Hence
//  * few heads are spread over many compute units (the split above, chosen by the launcher from the number of
//    heads), each workgroup fetching the chunk's shared operand block (one contiguous block per chunk, written
//    by the prep kernel) once for its NWC waves;
//  * the block goes through LDS.  Three LDS slots rotate with ONE LDS-only barrier per chunk (global loads stay
//    in flight across it):
//       step t:  barrier                      block t+1 (written during step t-1) becomes visible
//                share of block t+2 -> slot (t+2) % 3          (its last readers finished before the barrier)
//                read the operands of the state update of chunk t from slot t % 3
//                phase 1: v_new (operands already in registers, read during step t-1)
//                read the phase-1 operands of chunk t+1 from slot (t+1) % 3
//                phase 2: state update
//    so every LDS read has a phase of matrix products between its issue and its first use;
//  * for 2-byte inputs, four "memory waves" per workgroup do nothing but move data: they hold the register ring
//    of block shares (6 chunks in flight), hand them to LDS, and copy the results, which the computing waves
//    leave in an LDS outbox laid out like the chunk's record in global memory, out to global memory a step later.
//    The computing waves then touch global memory only for the few tiles that are theirs alone (rows of do in the
//    reverse scan; tiles of u^T and v^T in the forward scans, and for K = 64 these too travel through LDS with the
//    block).  Without memory waves (fp32 inputs, or eight computing waves) the computing waves do all of that
//    themselves.
#pragma once
#include "hdla_common.cuh"
#include "scan_shapes.h"

namespace hdla {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// workgroup barrier that orders LDS accesses only: global loads issued before it may still be outstanding
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

constexpr int NSLOT = 3;

template <typename T, int K, int V, int NWC> struct ScanCfg {
    static constexpr int VT = V / 16, SPLIT = VT / NWC;   // workgroups per head
    static constexpr int KB = K * (int)sizeof(T);         // bytes of one operand row
    static constexpr int NM = (sizeof(T) == 2 && NWC <= 4) ? 4 : 0;   // memory waves
    static constexpr int THREADS = 64 * (NWC + NM);
    static constexpr int NLD = NM ? NM : NWC;             // waves that split the loading of a block
    // forward scans with memory waves (rows of 128 bytes: the larger ones have no registers to spare): the tiles of
    // u^T and v^T of the workgroup's column blocks travel through LDS with the shared block (appended to it), so
    // that the computing waves issue no global loads at all
    static constexpr int OWN_UT = (NM && KB <= 128) ? NWC * PAIR * (int)sizeof(T) : 0, OWN_VTT = (NM && KB <= 128) ? NWC * TILE * (int)sizeof(T) : 0;
    static constexpr int OWN_FWD = (OWN_UT + OWN_VTT + 1023) & ~1023;
    // Depth of the register ring of block shares (chunks in flight from global memory) and of the computing
    // waves' own tiles; multiples of the number of slots so that slot numbers are static in the unrolled loops;
    // 0: no ring, one chunk at a time.
    static constexpr int DR_SHARE = NM ? 6 : (KB <= 128 ? 6 : KB <= 256 ? 3 : 0);
    static constexpr int DR_OWN = NM ? (KB <= 128 ? 6 : 3) : DR_SHARE;
    // Whether LDS reads are issued a phase ahead of their use as described above, or left where the compiler
    // puts them (the shapes whose operands would not fit the register file twice over) ...
    static constexpr bool pipelined(bool with_o) { return KB <= 128 || (KB <= 256 && !(NWC == 8 && with_o)); }
    // ... and whether that includes the operands of the state update
    static constexpr bool early_update_reads(bool with_o) { return KB <= 128 || (KB <= 256 && NWC <= 4 && (NM == 0 || with_o)); }
};

// A shared operand block as the loading waves see it: NI pieces of 1 KiB, lane l taking 16 bytes of each.  The
// first NT pieces hold tiles that are handed to LDS transposed, so a lane must hold whole fragments of them: for
// 2-byte elements a piece is a tile pair in its stored order; for 4-byte elements a piece is one tile of a pair,
// 16 of every 32 bytes.
template <int ES> __device__ __forceinline__ int piece_off(int i, int l, bool tiles) {
    if (ES == 4 && tiles) return (i >> 1) * 2048 + l * 32 + (i & 1) * 16;
    return i * 1024 + l * 16;
}
// the whole block is contiguous in global memory (forward scans)
struct BlockOne {
    const char* p;
    __device__ __forceinline__ const char* piece(int i, int l, bool) const { return p + i * 1024 + l * 16; }
};
// forward scan with memory waves: the block, then the workgroup's tiles of u^T, then those of v^T (the last piece may
// reach past them: those lanes read inside the tiles again, what they leave in LDS is never looked at)
template <int NIB, int UTB, int VTB> struct BlockFwd {
    const char *b, *ut, *vtt;
    __device__ __forceinline__ const char* piece(int i, int l, bool) const {
        if (i < NIB) return b + i * 1024 + l * 16;
        const int off = (i - NIB) * 1024 + l * 16;
        if (off < UTB) return ut + off;
        return vtt + (off - UTB) % VTB;
    }
};
// reverse scan: W and BGT (NIF pieces) and the piece holding EGL come from the forward-scan block of the (chunk,
// head), the rest is the reverse-scan block
template <typename T, int K> struct BlockTwo {
    const char *f, *r;
    __device__ __forceinline__ const char* piece(int i, int l, bool tiles) const {
        constexpr SlotB S = slot_bwd(K, sizeof(T));
        static_assert(S.EGL_SRC % 1024 == 0, "EGL starts a piece");
        if (i < S.NIF) return f + piece_off<sizeof(T)>(i, l, tiles);
        if (i == S.NIF) return f + S.EGL_SRC + l * 16;
        return r + (i - S.NIF - 1) * 1024 + l * 16;
    }
};

// 16 bytes of fragments of type T, each tile transposed (a product with the identity: exact)
template <typename T> __device__ __forceinline__ i32x4 transpose_piece(i32x4 x) {
    const Frag<T> ident = ident_frag<T>();
    if constexpr (sizeof(T) == 2) {
        const s16x8 y = __builtin_bit_cast(s16x8, x);
        Frag<T> f0, f1;
        f0.v = __builtin_shufflevector(y, y, 0, 1, 2, 3);
        f1.v = __builtin_shufflevector(y, y, 4, 5, 6, 7);
        f0 = transpose(f0, ident);
        f1 = transpose(f1, ident);
        return __builtin_bit_cast(i32x4, __builtin_shufflevector(f0.v, f1.v, 0, 1, 2, 3, 4, 5, 6, 7));
    } else {
        Frag<T> f;
        f.v = __builtin_bit_cast(f32x4, x);
        return __builtin_bit_cast(i32x4, transpose(f, ident).v);
    }
}

// one wave's share of a shared operand block: the pieces w, w+NLD, ... of its NI pieces
template <typename T, int NI, int NLD, int NT = 0> struct Share {
    static constexpr int CNT = (NI + NLD - 1) / NLD;
    static_assert(NT % NLD == 0 && NT < NI, "whether a piece is transposed must not depend on the wave");
    i32x4 a[CNT];
    template <typename Blk> __device__ __forceinline__ void load(const Blk& blk, int w) {
        const int l = lane_id();
#pragma unroll
        for (int j = 0; j < CNT; ++j) {
            const int i = min(w + j * NLD, NI - 1);       // the last pieces may be fetched twice; never out of range
            a[j] = *reinterpret_cast<const i32x4*>(blk.piece(i, l, j * NLD < NT));
        }
    }
    __device__ __forceinline__ void to_lds(char* slot, int w) const {
        const int l = lane_id();
#pragma unroll
        for (int j = 0; j < CNT; ++j) {
            const int i = min(w + j * NLD, NI - 1);
            const bool tiles = j * NLD < NT;
            *reinterpret_cast<i32x4*>(slot + piece_off<sizeof(T)>(i, l, tiles)) = tiles ? transpose_piece<T>(a[j]) : a[j];
        }
    }
};

// A memory wave.  blk(t): block of step t (clamped to the last step by the caller); out(t): copy the outbox of
// step t to global memory.  Barriers: one closing the prologue, one per step, one handing over the last outbox;
// the computing waves execute exactly the same sequence.
template <typename T, int NI, int NM, int DR, int SLOT, int NT, typename BlkFn, typename OutFn>
__device__ __forceinline__ void memory_wave(char* smem, int nsteps, int hw, BlkFn blk, OutFn out) {
    static_assert(DR % NSLOT == 0 && DR >= NSLOT, "ring depth must be a multiple of the slot count");
    Share<T, NI, NM, NT> sh[DR];
#pragma unroll
    for (int d = 0; d < DR; ++d) sh[d].load(blk(d), hw);
    sh[0].to_lds(smem, hw);
    sh[1].to_lds(smem + SLOT, hw);
    sh[0].load(blk(DR), hw);
    sh[1].load(blk(DR + 1), hw);
    lds_barrier();
    const int nfull = nsteps / DR;
#pragma unroll 1
    for (int gi = 0; gi < nfull; ++gi) {
#pragma unroll
        for (int j = 0; j < DR; ++j) {
            const int t = gi * DR + j;
            lds_barrier();
            sh[(j + 2) % DR].to_lds(smem + ((j + 2) % NSLOT) * SLOT, hw);
            sh[(j + 2) % DR].load(blk(t + 2 + DR), hw);
            if (t > 0) out(t - 1);
        }
    }
#pragma unroll 1
    for (int t = nfull * DR; t < nsteps; ++t) {           // fewer than DR steps left: one block at a time
        lds_barrier();
        Share<T, NI, NM, NT> tmp;
        tmp.load(blk(t + 2), hw);
        if (t > 0) out(t - 1);
        tmp.to_lds(smem + ((t + 2) % NSLOT) * SLOT, hw);
    }
    lds_barrier();
    out(nsteps - 1);
}

// LDS of a scan workgroup: the three operand slots, then (with memory waves) two outboxes.  What an outbox holds:
//   OUT_O      forward pass: the workgroup's 16 x (16 NWC) piece of the output rows, padded by 16 bytes a row
//              against bank conflicts;
//   OUT_STATE  forward scan of the backward pass: the workgroup's part of the chunk's state checkpoint,
//              [K/32][NWC] tile pairs (1 KiB a pair for 2-byte elements).  v_new is not checkpointed: the
//              chunk_grad kernel rebuilds it from this checkpoint, w and u;
//   OUT_GRAD   reverse scan: the same for dS, followed by [NWC] tile pairs of dv_new.
enum ScanOut { OUT_O, OUT_STATE, OUT_GRAD };
template <typename T, int K, int V, int NWC, int SLOT_, ScanOut OUT> struct ScanLds {
    static constexpr int ES = sizeof(T), NM = ScanCfg<T, K, V, NWC>::NM, SLOT = SLOT_;
    static constexpr int OROW = 16 * NWC * ES + 16;
    static constexpr int OB_HC = (K / 32) * NWC * PAIR * ES;
    static constexpr int OB = OUT == OUT_O ? CH * OROW : OUT == OUT_STATE ? OB_HC : OB_HC + NWC * PAIR * ES;
    static constexpr int BYTES = NSLOT * SLOT + (NM ? 2 * OB : 0);
};

// ---- forward -------------------------------------------------------------------------------------------------
template <typename T, int K, int V, int NWC, bool WRITE_O>
__device__ __forceinline__ void scan_fwd_body(const ChunkArgs<T>& p, char* smem, int n, int split) {
    typedef ScanCfg<T, K, V, NWC> C;
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NM = C::NM, ES = sizeof(T);
    constexpr BlkF B = blk_fwd(K, sizeof(T), WRITE_O);
    constexpr bool PIPE = C::pipelined(WRITE_O);
    constexpr bool PIPE_UPD = PIPE && C::early_update_reads(WRITE_O);
    constexpr int NIB = B.SIZE / 1024, SLOT = B.SIZE + C::OWN_FWD, NI = SLOT / 1024;
    constexpr bool OWN_LDS = C::OWN_FWD > 0;
    typedef ScanLds<T, K, V, NWC, SLOT, WRITE_O ? OUT_O : OUT_STATE> L;
    constexpr int OROW = L::OROW, OB_HC = L::OB_HC, OB = L::OB;
    char* const outbox = smem + NSLOT * SLOT;

    const int h = blockIdx.x;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int vt0 = split * NWC;                          // first column block of this workgroup
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const int nchunks = c1 - c0, last = c1 - 1;
    // block of step t; steps past the end of the sequence are clamped, so every load is unconditional (a load
    // that may or may not have been issued would make the compiler wait for all outstanding loads)
    auto blk = [&](int t) __attribute__((always_inline)) {
        const int64_t chw = chw0 + min(c0 + t, last);
        // (the forward pass's blocks are B.SIZE apart; those the backward pass reads may be a forward pass's, further apart)
        const char* b = reinterpret_cast<const char*>(p.ws.W) + chw * (WRITE_O ? B.SIZE : p.ws.sa_stride);
        if constexpr (OWN_LDS)
            return BlockFwd<NIB, C::OWN_UT, C::OWN_VTT>{b, reinterpret_cast<const char*>(p.ws.UT + (chw * VT + vt0) * PAIR),
                                                        reinterpret_cast<const char*>(p.ws.VTT + (chw * VT + vt0) * TILE)};
        else
            return BlockOne{b};
    };

    if (NM && wv >= NWC) {
        if (nchunks <= 0) return;
        const int hw = wv - NWC;
        memory_wave<T, NI, NM ? NM : 1, NM ? C::DR_SHARE : NSLOT, SLOT, 0>(smem, nchunks, hw, blk, [&](int t) __attribute__((always_inline)) {
            const int cid = c0 + t;
            const char* ob = outbox + (t & 1) * OB;
            if (WRITE_O) {
                // rows of o: 16-byte pieces, LPR lanes a row
                constexpr int LPR = 16 * NWC * ES / 16, RPI = 64 / LPR;
                const int64_t tok0 = bos + (int64_t)t * CH;
                const int len = (int)min((int64_t)CH, eos - tok0);
#pragma unroll
                for (int r0 = hw * RPI; r0 < CH; r0 += (NM ? NM : 1) * RPI) {
                    const int r = r0 + l / LPR, e = (l % LPR) * 16;
                    if (r < len) {                        // also keeps lanes beyond the 16 rows inside the outbox
                        const i32x4 x = *reinterpret_cast<const i32x4*>(ob + r * OROW + e);
                        *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(p.o + ((tok0 + r) * H + h) * V + 16 * vt0) + e) = x;
                    }
                }
            } else {
                char* hc = reinterpret_cast<char*>(p.ws.HC + (chw0 + cid) * (K * V) + vt0 * PAIR);
                constexpr int NP = OB / 1024;
#pragma unroll
                for (int j = 0; j < (NP + (NM ? NM : 1) - 1) / (NM ? NM : 1); ++j) {
                    const int i = hw + j * (NM ? NM : 1);
                    if (i < NP)
                        *reinterpret_cast<i32x4*>(hc + ((i / NWC) * VT + i % NWC) * 1024 + l * 16) =
                            *reinterpret_cast<const i32x4*>(ob + i * 1024 + l * 16);
                }
            }
        });
        return;
    }

    // ---- computing wave
    const int vt = vt0 + wv;
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
    struct Own { Frag<T> ut[2], vtt; };                   // the tiles only this wave reads (from LDS where they travel with the block)
    auto load_own = [&](Own& o, int t) __attribute__((always_inline)) {
        if constexpr (!OWN_LDS) {
            const int64_t chw = chw0 + min(c0 + t, last);
            ld_pair(p.ws.UT + (chw * VT + vt) * PAIR, o.ut[0], o.ut[1]);
            o.vtt = ld_tile(p.ws.VTT + (chw * VT + vt) * TILE);
        }
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
    // that go to global memory into the outbox `ob` (when there are memory waves)
    auto step = [&](const char* slot, const char* slot_next, char* ob, Own own, int t) __attribute__((always_inline)) {
        const int cid = c0 + t;
        const int64_t chw = chw0 + cid;
        const int64_t tok0 = bos + (int64_t)t * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        if constexpr (OWN_LDS) {
            ld_pair(reinterpret_cast<const T*>(slot + B.SIZE) + wv * PAIR, own.ut[0], own.ut[1]);
            own.vtt = ld_tile(reinterpret_cast<const T*>(slot + B.SIZE + C::OWN_UT) + wv * TILE);
        }
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
            // checkpoint of the entering state, as the fragments held here (tile pairs, 16 bytes per lane, whole
            // cache lines): the chunk_grad kernel turns them the way it needs them
            T* hc = NM ? reinterpret_cast<T*>(ob) + wv * PAIR : p.ws.HC + chw * (K * V) + vt * PAIR;
            constexpr int HSTR = (NM ? NWC : VT) * PAIR;  // elements between the pairs of consecutive channel tiles
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) st_pair2(hc + kp * HSTR, sb[2 * kp], sb[2 * kp + 1]);
        }
        if (WRITE_O) {
            o = mm(aqb[0], vnb[0], o);
            o = mm(aqb[1], vnb[1], o);
            if (NM) st_frag(reinterpret_cast<T*>(ob + c * OROW) + 16 * wv + 4 * g, to_frag<T>(o));
            else if (c < len) st_frag(p.o + ((tok0 + c) * H + h) * V + 16 * vt + 4 * g, to_frag<T>(o));
            // the output leaves for the outbox before the state update below, not after it: the barrier that ends the step
            // waits for this LDS write, and behind the update's products the wait is free
            if (NM && PIPE) __builtin_amdgcn_sched_barrier(0);
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
        constexpr int DRO = C::DR_OWN, DRS = NM ? 0 : C::DR_SHARE;   // without memory waves both rings are one
        int done = 0;
        if constexpr (DRO > 0) {
            Share<T, NI, NWC> sh[DRS ? DRS : 1];
            Own own[DRO];
#pragma unroll
            for (int d = 0; d < DRO; ++d) {
                if (DRS) sh[DRS ? d : 0].load(blk(d), wv);
                load_own(own[d], d);
            }
            if (DRS) {
                sh[0].to_lds(smem, wv);
                sh[DRS ? 1 : 0].to_lds(smem + SLOT, wv);
                sh[0].load(blk(DRS), wv);
                sh[DRS ? 1 : 0].load(blk(DRS + 1), wv);
            }
            lds_barrier();
            if (PIPE) read_w_all(smem);
            const int nfull = nchunks / DRO;
#pragma unroll 1
            for (int gi = 0; gi < nfull; ++gi) {
#pragma unroll
                for (int j = 0; j < DRO; ++j) {            // DRO is a multiple of NSLOT: step gi*DRO+j uses slot j % 3
                    const int t = gi * DRO + j;
                    lds_barrier();
                    if (DRS) {
                        sh[DRS ? (j + 2) % DRO : 0].to_lds(smem + ((j + 2) % NSLOT) * SLOT, wv);
                        sh[DRS ? (j + 2) % DRO : 0].load(blk(t + 2 + DRS), wv);
                    }
                    step(smem + (j % NSLOT) * SLOT, smem + ((j + 1) % NSLOT) * SLOT, outbox + (t & 1) * OB, own[j], t);
                    // refilled only after the last use: a register that is loaded while its old value is still
                    // live needs a copy, and the copy would wait for the load just issued
                    load_own(own[j], t + DRO);
                }
            }
            done = nfull * DRO;
        } else {
            Share<T, NI, NWC> tmp;
            tmp.load(blk(0), wv);
            tmp.to_lds(smem, wv);
            tmp.load(blk(1), wv);
            tmp.to_lds(smem + SLOT, wv);
            lds_barrier();
            if (PIPE) read_w_all(smem);
        }
        // what is left (fewer than a ring of chunks, or all of them without a ring): one at a time, same protocol
        if (done < nchunks) {
            Own cur;
            load_own(cur, done);
#pragma unroll 1
            for (int t = done; t < nchunks; ++t) {
                lds_barrier();
                Share<T, NI, NWC> tmp;
                if (!NM) tmp.load(blk(t + 2), wv);
                Own nxt;
                load_own(nxt, t + 1);
                step(smem + (t % NSLOT) * SLOT, smem + ((t + 1) % NSLOT) * SLOT, outbox + (t & 1) * OB, cur, t);
                if (!NM) tmp.to_lds(smem + ((t + 2) % NSLOT) * SLOT, wv);
                cur = nxt;
            }
        }
        if (NM) lds_barrier();                            // hands the last outbox to the memory waves
    }
    if (p.ht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
// Step t handles chunk c1-1-t.
template <typename T, int K, int V, int NWC>
__device__ __forceinline__ void scan_bwd_body(const ChunkArgs<T>& p, char* smem, int n, int split) {
    typedef ScanCfg<T, K, V, NWC> C;
    constexpr int KT = K / 16, KT2 = KT / 2, VT = V / 16, NM = C::NM, ES = sizeof(T);
    // LDS slot: [BG | WT] (BGT and W of the forward-scan block, transposed on their way in) | EGL | QGT | AQBT
    constexpr SlotB B = slot_bwd(K, sizeof(T));
    constexpr int SBWD = blk_bwd(K, sizeof(T)).SIZE, NT = B.NIF;
    const int SFWD = p.ws.sa_stride;
    constexpr bool PIPE = C::pipelined(false);
    constexpr bool PIPE_UPD = PIPE && C::early_update_reads(false);
    constexpr int NI = B.SIZE / 1024, SLOT = B.SIZE;
    typedef ScanLds<T, K, V, NWC, SLOT, OUT_GRAD> L;
    constexpr int OB_HC = L::OB_HC, OB = L::OB;
    char* const outbox = smem + NSLOT * SLOT;

    const int h = blockIdx.x;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int vt0 = split * NWC;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    const int64_t chw0 = (int64_t)h * p.st.nch;
    const int nchunks = c1 - c0, first = c1 - 1;
    auto blk = [&](int t) __attribute__((always_inline)) {
        const int64_t slot = chw0 + max(first - t, c0);
        return BlockTwo<T, K>{reinterpret_cast<const char*>(p.ws.W) + slot * SFWD, reinterpret_cast<const char*>(p.ws.QGT) + slot * SBWD};
    };

    if (NM && wv >= NWC) {
        if (nchunks <= 0) return;
        const int hw = wv - NWC;
        memory_wave<T, NI, NM ? NM : 1, NM ? C::DR_SHARE : NSLOT, SLOT, NT>(smem, nchunks, hw, blk, [&](int t) __attribute__((always_inline)) {
            const int cid = first - t;
            const char* ob = outbox + (t & 1) * OB;
            char* hc = reinterpret_cast<char*>(p.ws.DHC + (chw0 + cid) * (K * V) + vt0 * PAIR);
            char* vn = reinterpret_cast<char*>(p.ws.DVN + (chw0 + cid) * (2 * CH * V) + vt0 * PAIR);
            constexpr int NP = OB / 1024, NPH = OB_HC / 1024;
#pragma unroll
            for (int j = 0; j < (NP + (NM ? NM : 1) - 1) / (NM ? NM : 1); ++j) {
                const int i = hw + j * (NM ? NM : 1);
                if (i < NP) {
                    char* dst = i < NPH ? hc + ((i / NWC) * VT + i % NWC) * 1024 : vn + (i - NPH) * 1024;
                    *reinterpret_cast<i32x4*>(dst + l * 16) = *reinterpret_cast<const i32x4*>(ob + i * 1024 + l * 16);
                }
            }
        });
        return;
    }

    const int vt = vt0 + wv;
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
    // rows of do; rows past the end of a ragged chunk alias its last row and are zeroed where used
    auto load_own = [&](Frag<T>& don, int t) __attribute__((always_inline)) {
        const int cid = max(first - t, c0);
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        don = ld_frag(p.dout + ((tok0 + min(c, len - 1)) * H + h) * V + 16 * vt + 4 * g);
    };

    Frag<T> aq[2], bg[2][KT];                             // phase-1 operands; when pipelined, read a step ahead
    auto read_bg = [&](const char* slot, int kp) __attribute__((always_inline)) {
        const T* sBG = reinterpret_cast<const T*>(slot + B.BGT);
        ld_pair(sBG + (0 * KT2 + kp) * PAIR, bg[0][2 * kp], bg[0][2 * kp + 1]);
        ld_pair(sBG + (1 * KT2 + kp) * PAIR, bg[1][2 * kp], bg[1][2 * kp + 1]);
    };
    auto read_p1_all = [&](const char* slot) __attribute__((always_inline)) {
        ld_pair(reinterpret_cast<const T*>(slot + B.AQBT), aq[0], aq[1]);
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) read_bg(slot, kp);
    };

    auto step = [&](const char* slot, const char* slot_next, char* ob, Frag<T> don, int t) __attribute__((always_inline)) {
        const int cid = first - t;
        const int64_t chw = chw0 + cid;
        const T* sWT = reinterpret_cast<const T*>(slot + B.W);
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
        T* dhc = NM ? reinterpret_cast<T*>(ob) + wv * PAIR : p.ws.DHC + chw * (K * V) + vt * PAIR;
        T* dvp = NM ? reinterpret_cast<T*>(ob + OB_HC) + wv * PAIR : p.ws.DVN + chw * (2 * CH * V) + vt * PAIR;
        constexpr int HSTR = (NM ? NWC : VT) * PAIR;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) st_pair2(dhc + kp * HSTR, dsb[2 * kp], dsb[2 * kp + 1]);
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
        constexpr int DRO = C::DR_OWN, DRS = NM ? 0 : C::DR_SHARE;
        int done = 0;
        if constexpr (DRO > 0) {
            Share<T, NI, NWC, NT> sh[DRS ? DRS : 1];
            Frag<T> own[DRO];
#pragma unroll
            for (int d = 0; d < DRO; ++d) {
                if (DRS) sh[DRS ? d : 0].load(blk(d), wv);
                load_own(own[d], d);
            }
            if (DRS) {
                sh[0].to_lds(smem, wv);
                sh[DRS ? 1 : 0].to_lds(smem + SLOT, wv);
                sh[0].load(blk(DRS), wv);
                sh[DRS ? 1 : 0].load(blk(DRS + 1), wv);
            }
            lds_barrier();
            if (PIPE) read_p1_all(smem);
            const int nfull = nchunks / DRO;
#pragma unroll 1
            for (int gi = 0; gi < nfull; ++gi) {
#pragma unroll
                for (int j = 0; j < DRO; ++j) {
                    const int t = gi * DRO + j;
                    lds_barrier();
                    if (DRS) {
                        sh[DRS ? (j + 2) % DRO : 0].to_lds(smem + ((j + 2) % NSLOT) * SLOT, wv);
                        sh[DRS ? (j + 2) % DRO : 0].load(blk(t + 2 + DRS), wv);
                    }
                    step(smem + (j % NSLOT) * SLOT, smem + ((j + 1) % NSLOT) * SLOT, outbox + (t & 1) * OB, own[j], t);
                    load_own(own[j], t + DRO);             // after the last use of the old value: no copy, no wait
                }
            }
            done = nfull * DRO;
        } else {
            Share<T, NI, NWC, NT> tmp;
            tmp.load(blk(0), wv);
            tmp.to_lds(smem, wv);
            tmp.load(blk(1), wv);
            tmp.to_lds(smem + SLOT, wv);
            lds_barrier();
            if (PIPE) read_p1_all(smem);
        }
        if (done < nchunks) {
            Frag<T> cur;
            load_own(cur, done);
#pragma unroll 1
            for (int t = done; t < nchunks; ++t) {
                lds_barrier();
                Share<T, NI, NWC, NT> tmp;
                if (!NM) tmp.load(blk(t + 2), wv);
                Frag<T> nxt;
                load_own(nxt, t + 1);
                step(smem + (t % NSLOT) * SLOT, smem + ((t + 1) % NSLOT) * SLOT, outbox + (t & 1) * OB, cur, t);
                if (!NM) tmp.to_lds(smem + ((t + 2) % NSLOT) * SLOT, wv);
                cur = nxt;
            }
        }
        if (NM) lds_barrier();
    }
    if (p.dh0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.dh0[soff + (int64_t)(16 * kt + 4 * g + i) * V] = dS[kt][i];
    }
}

// ---- kernels ---------------------------------------------------------------------------------------------------
// grid = (H, directions * SPLIT, N): blockIdx.y = direction * SPLIT + split; blockIdx.z counts the sequences, packed
// ones from the longest down.  Workgroups start in the order of their linear index (x fastest): the workgroups of one
// (sequence, head) are H apart, which puts them on the same XCD (and its L2, where they share the chunk blocks) when H
// is a multiple of 8, and when the launch has more workgroups than the device holds at once, the long sequences,
// which decide when the launch ends, start first and the short ones fill in behind them.
__device__ __forceinline__ int scan_sequence(const SeqTab& st) { return st.cu ? st.order[blockIdx.z] : (int)blockIdx.z; }
template <typename T, int K, int V, int NWC, bool WRITE_O>
__global__ __launch_bounds__((ScanCfg<T, K, V, NWC>::THREADS)) void scan_fwd_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[ScanLds<T, K, V, NWC, blk_fwd(K, sizeof(T), WRITE_O).SIZE + ScanCfg<T, K, V, NWC>::OWN_FWD, WRITE_O ? OUT_O : OUT_STATE>::BYTES];
    scan_fwd_body<T, K, V, NWC, WRITE_O>(p, smem, scan_sequence(p.st), blockIdx.y);
}
template <typename T, int K, int V, int NWC>
__global__ __launch_bounds__((ScanCfg<T, K, V, NWC>::THREADS)) void scan_bwd_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[ScanLds<T, K, V, NWC, slot_bwd(K, sizeof(T)).SIZE, OUT_GRAD>::BYTES];
    scan_bwd_body<T, K, V, NWC>(p, smem, scan_sequence(p.st), blockIdx.y);
}
// Both scans of the backward pass in one launch: they depend on the prep kernel only, not on each other.
template <typename T, int K, int V, int NWC>
__global__ __launch_bounds__((ScanCfg<T, K, V, NWC>::THREADS)) void scan_pair_kernel(ChunkArgs<T> p) {
    constexpr int NF = ScanLds<T, K, V, NWC, blk_fwd(K, sizeof(T), false).SIZE + ScanCfg<T, K, V, NWC>::OWN_FWD, OUT_STATE>::BYTES;
    constexpr int NB = ScanLds<T, K, V, NWC, slot_bwd(K, sizeof(T)).SIZE, OUT_GRAD>::BYTES;
    constexpr int SPLIT = ScanCfg<T, K, V, NWC>::SPLIT;
    __shared__ __attribute__((aligned(16))) char smem[NF > NB ? NF : NB];
    const int n = scan_sequence(p.st);
    if (blockIdx.y < SPLIT) scan_fwd_body<T, K, V, NWC, false>(p, smem, n, blockIdx.y);
    else scan_bwd_body<T, K, V, NWC>(p, smem, n, blockIdx.y - SPLIT);
}

// ---- launchers -------------------------------------------------------------------------------------------------
template <typename T, int K, int V, int NWC>
static hipError_t launch_scan_nwc(const ChunkArgs<T>& a, ScanKind kind, hipStream_t stream) {
    typedef ScanCfg<T, K, V, NWC> C;
    dim3 grid(a.H, C::SPLIT * (kind == SCAN_PAIR ? 2 : 1), a.st.N), block(C::THREADS);
    switch (kind) {
        case SCAN_FWD_O: hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, NWC, true>), grid, block, 0, stream, a); break;
        case SCAN_FWD: hipLaunchKernelGGL((scan_fwd_kernel<T, K, V, NWC, false>), grid, block, 0, stream, a); break;
        case SCAN_BWD: hipLaunchKernelGGL((scan_bwd_kernel<T, K, V, NWC>), grid, block, 0, stream, a); break;
        case SCAN_PAIR: hipLaunchKernelGGL((scan_pair_kernel<T, K, V, NWC>), grid, block, 0, stream, a); break;
    }
    return hipGetLastError();
}

// Workgroups per head: as many as keep the whole launch within the compute units of the device (one workgroup per
// unit: what a split buys is memory throughput), 2-byte inputs only.
constexpr int SCAN_TARGET_WORKGROUPS = 256;
template <typename T, int K, int V>
hipError_t launch_scan_shape(const ChunkArgs<T>& a, ScanKind kind, hipStream_t stream) {
    constexpr int VT = V / 16;
    if constexpr (sizeof(T) == 2) {
        const int lanes = a.H * a.st.N * (kind == SCAN_PAIR ? 2 : 1);
        if (lanes * 4 <= SCAN_TARGET_WORKGROUPS) return launch_scan_nwc<T, K, V, VT / 4>(a, kind, stream);
        // eight computing waves leave no room for memory waves: V = 128 is always split at least in two
        if (lanes * 2 <= SCAN_TARGET_WORKGROUPS || VT == 8) return launch_scan_nwc<T, K, V, VT / 2>(a, kind, stream);
        if constexpr (VT == 8) return hipErrorInvalidValue;   // not reached
        else return launch_scan_nwc<T, K, V, VT>(a, kind, stream);
    } else {
        return launch_scan_nwc<T, K, V, VT>(a, kind, stream);
    }
}

}  // namespace hdla
