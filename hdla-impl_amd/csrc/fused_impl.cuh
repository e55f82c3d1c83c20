// Fused chunk kernels: the per-chunk preparation (cumulative decays, score tiles, (I - A_ab)^-1, w, u, gated copies:
// HRDPLR/fwd_triton.py:22-790 and fla's chunk_rwkv6_fwd_cumsum) and the inter-chunk state scan that consumes it
// (HRDPLR/fwd_triton.py:808-1095, HRDPLR/bwd_triton.py:127-222) in ONE kernel, so that what the preparation produces
// for the scan -- 14 to 20 KB per (16-token chunk, head) -- goes through LDS and never through HBM.
//
// Work division.  A workgroup owns one (sequence, head, time segment): the chunks of a sequence are cut into `nseg`
// consecutive segments so that few (sequence, head) pairs still fill the device.  It has
//   * FNP = 4 pairs of producer waves.  Pair p prepares the chunks p, p+4, ... of the segment and leaves the operands in
//     LDS slot p.  The two waves of a pair take two of the four channel tiles and half of the value tiles each; one of
//     them (the pair's lead) also adds up the two waves' parts of the score tiles and solves for (I - A_ab)^-1;
//   * V/16 consumer waves.  Consumer j owns column block j of the fp32 state for the whole segment, in registers, and
//     walks the chunks in order, exactly as the stand-alone scan kernels do.
// A segment other than the first does not know the state that enters it.  The state leaving a chunk is affine in the
// state entering it, so such a segment runs from zero and, beside it, carries the K x K transition matrix M (the same
// update applied to K more columns that start from the identity: consumer j also owns column block j of M).  What the
// chunk's output gains per unit of entering state, G = (qg + A_qb w) M (16 x K), comes out of the same products.
//   forward pass:   o_local and G go to the workspace; fixup_kernel chains the segments' (M, S_local) into the true
//                   entering states and adds G S_in.
//   backward pass:  the entering states are known (kept by the forward pass, or re-derived by a summary-only pass), so
//                   the state checkpoints are exact; M and R = sum_t G_t^T do_t give the gradient entering each
//                   segment from the right, d S_in(s) = M_s^T d S_in(s+1) + R_s, which the reverse kernel's consumers
//                   chain themselves before they start.
//
// Synchronisation.  Producers and consumers run at their own pace; a slot is handed over through two counters in LDS
// that only ever grow: ready[p] (+1 per wave of pair p and chunk completed) and consumed[p] (consumer-steps finished on
// slot p); the waves of a pair hand each other the parts and the inverse the same way (part[p], inv[p]).
// Waiting is polling with s_sleep; every wait is bounded (FUSED_SPIN_LIMIT polls), and a wave that runs into the bound
// raises an abort flag that ends every other wave's waits as well and is reported through FusedArgs::err, so the grid
// always drains.  There are no workgroup barriers after the first.
#pragma once
#include "hdla_common.cuh"
#include "fused_shapes.h"

namespace hdla {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int FNP = 4;                    // producer pairs = LDS slots
constexpr int FLDP = 36;                  // padded row length of the 32 x 32 matrices of the triangular solve
constexpr int FUSED_SPIN_LIMIT = 1 << 20; // polls of ~256 cycles: a tenth of a second, four orders above any real wait
// What a wave that gave up writes to FusedArgs::err (+1 producer, +2 forward consumer, +3 reverse consumer).  The word is
// never cleared (that would take a launch of its own): it is a diagnostic that reads as this pattern only after an
// abort, or by a one-in-a-billion coincidence with what the caller's memory held before.
constexpr int FUSED_ABORTED = 0x48444c00;

// chunk range [s0, s1) of time segment `seg` of sequence n
__device__ __forceinline__ void seg_range(const SeqTab& st, int n, int nseg, int seg, int& s0, int& s1) {
    int c0, c1;
    seq_chunks(st, n, c0, c1);
    const int len = (c1 - c0 + nseg - 1) / nseg;
    s0 = min(c0 + seg * len, c1);
    s1 = min(s0 + len, c1);
}

// LDS of a fused workgroup (byte offsets): per producer one slot = [operands | outbox | solver scratch], then the flags
template <typename T, int K, int V, int MODE> struct FusedLds {
    static constexpr int ES = sizeof(T), TB = TILE * ES, KT = K / 16, VT = V / 16;
    static constexpr bool REV = MODE == FUSED_REV;
    static constexpr BlkF BF = blk_fwd(K, ES, true);
    static constexpr SlotB SB = slot_bwd(K, ES);
    // forward direction: the forward-scan block, then u^T (VT tile pairs), v^T (VT tiles), and in checkpoint mode do^T
    // (VT tiles) and the inverse for chunk_grad
    static constexpr int UT = BF.SIZE, VTT = UT + 2 * VT * TB, DOT_F = VTT + VT * TB;
    // reverse direction: the reverse-scan slot, then do^T
    static constexpr int DOT = REV ? SB.SIZE : DOT_F;
    static constexpr int TMB = DOT_F + VT * TB;          // checkpoint mode: (I - A_ab)^-1 as chunk_grad reads it (2 tile pairs)
    static constexpr int OPER = REV ? SB.SIZE + VT * TB : (MODE == FUSED_CKPT ? TMB + 4 * TB : DOT_F);
    // outbox of the forward pass: 16 rows of o (fp32 in segments > 0, element type in segment 0) and 16 rows of G
    static constexpr int OROW = V * 4 + 16, GROW = K * ES + 16;
    static constexpr int OBOX = OPER, GBOX = OBOX + (MODE == FUSED_FWD ? CH * OROW : 0);
    static constexpr int SOLVE = GBOX + (MODE == FUSED_FWD ? CH * GROW : 0);
    static constexpr int SLOT = SOLVE + 2 * 32 * FLDP * 4;
    // int ready[4], consumed[4], abort, -, -, -, part[4], inv[4], strong[4] (per producer pair; see fused_producer), then
    // two counters of the reverse kernel's consumers (records staged, records used: fused_consumer_rev)
    static constexpr int FLAGS = FNP * SLOT;
    // reverse kernel: transition records of the segments to the right, as split operands, for the consumers' chain
    // (CHAIN_STAGE records of K x K at a time: every consumer wave needs them whole, each loads a quarter)
    static constexpr int CHAIN_STAGE = 2;
    static constexpr int CHAIN = FLAGS + 128;
    static constexpr int BYTES = CHAIN + (REV ? CHAIN_STAGE * 2 * KT * KT * TB : 0);
};

// ---- hand-over counters ------------------------------------------------------------------------------------------
__device__ __forceinline__ bool wait_ge(int* flag, int want, int* abort_flag) {
    int spins = 0;
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < want) {
        if (__hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0 || ++spins > FUSED_SPIN_LIMIT) {
            __hip_atomic_store(abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            return false;
        }
        __builtin_amdgcn_s_sleep(4);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return true;
}
// all LDS accesses of the wave so far are complete before the counter moves
__device__ __forceinline__ void signal_set(int* flag, int value) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    if (lane_id() == 0) __hip_atomic_store(flag, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void signal_add(int* flag) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    if (lane_id() == 0) __hip_atomic_fetch_add(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// the log-decay of four channels as it sits in memory (element type or fp32), converted and masked only where it is used
template <typename T, bool GKF32> struct GkRaw {
    typedef Frag<T> type;
    static __device__ __forceinline__ type load(const char* p) { return ld_frag(reinterpret_cast<const T*>(p)); }
    static __device__ __forceinline__ f32x4 value(type x, bool ok) { return ok ? to_f32(x) : zero4(); }
};
template <typename T> struct GkRaw<T, true> {
    typedef f32x4 type;
    static __device__ __forceinline__ type load(const char* p) { return *reinterpret_cast<const f32x4*>(p); }
    static __device__ __forceinline__ f32x4 value(type x, bool ok) { return ok ? x : zero4(); }
};

// F(I16) for lane (g, c), like ident_frag() but from the caller's lane coordinates
template <typename T> __device__ __forceinline__ Frag<T> ident_of(int g, int c) {
    f32x4 e;
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = (c == 4 * g + i) ? 1.f : 0.f;
    return to_frag<T>(e);
}

// ---- producers -----------------------------------------------------------------------------------------------------
// Everything of a chunk that does not depend on the state, by a PAIR of waves, into LDS slot `pp`.  Wave `half` of the
// pair takes the channel tiles 2 half, 2 half + 1 (one stored tile pair of every operand) and half of the value tiles.
// The score tiles are sums over all channels: the other wave hands its parts to the pair's `lead` wave through LDS, the
// lead solves the (small) triangular system and hands (I - A_ab)^-1 and A_ak back, and each forms w and u for its own
// tiles.  The formulas are the stand-alone prep kernel's (prep.hip); what differs from its one-wave form is the order
// in which the two halves of a score tile's sum over channels are added.
//
// One wave per chunk (the first form of this kernel) took 19,000 cycles a chunk, most of them waiting for its own
// previous instruction: alone on its SIMD nothing fills those gaps.  Two waves per chunk on three waves per SIMD do.
template <typename T, bool GKF32, int K, int V, int MODE, bool HD>
__device__ __forceinline__ void fused_producer(const FusedArgs<T>& a, char* smem, int n, int h, int seg, int s0, int s1, int pp, int half) {
    static_assert(K == 64 && sizeof(T) == 2 && V % 32 == 0, "a producer pair holds all channels of a chunk: K = 64, 2-byte elements");
    typedef FusedLds<T, K, V, MODE> L;
    constexpr bool REV = MODE == FUSED_REV, CKPT = MODE == FUSED_CKPT, FWD = MODE == FUSED_FWD;
    constexpr int KT = K / 16, VT = V / 16, KT2 = KT / 2, KH = 2, VH = VT / 2;
    constexpr BlkF BF = L::BF;
    constexpr SlotB SB = L::SB;
    const ChunkArgs<T>& p = a.c;
    char* slot = smem + pp * L::SLOT;
    // the pair's scratch: first the other wave's parts of the nine score tiles (fp32, 9 KiB); then, in the same bytes,
    // A_ab and its inverse for the solve; then the inverse and A_ak as operand tiles for the other wave
    float *sP, *sN, *sT;
    T* sPub;
    int* const flags = reinterpret_cast<int*>(smem + L::FLAGS);
    int* const f_ready = flags + pp, * const f_consumed = flags + 4 + pp, * const f_abort = flags + 8;
    int* const f_part = flags + 12 + pp, * const f_inv = flags + 16 + pp, * const f_strong = flags + 20 + pp;
    const bool lead = half == (pp >> 1);                  // spreads the leads over the SIMDs
    int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    const float scale = p.scale;
    const int nst = s1 - s0;
    const int kt0 = half * KH, vt0 = half * VH;
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    int c0, c1;
    seq_chunks(p.st, n, c0, c1);

    // rows of the previous chunk's results, left in the outbox by the consumers, out to global memory (forward pass);
    // each wave of the pair takes half of the rows
    auto copy_out = [&](int cid) __attribute__((always_inline)) {
        if constexpr (FWD) {
            // the lane's offsets below are formed afresh in every call: hoisted out of the chunk loop they would be held
            // in registers through all of it
            int l = lane_id();
            asm volatile("" : "+v"(l));
            const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
            const int len = (int)min((int64_t)CH, eos - tok0);
            const int64_t chw = (int64_t)h * p.st.nch + cid;
            const int rb = half * (CH / 2);
            if (seg == 0) {
                constexpr int LPR = V * (int)sizeof(T) / 16, RPI = 64 / LPR;
#pragma unroll
                for (int r0 = 0; r0 < CH / 2; r0 += RPI) {
                    const int r = rb + r0 + l / LPR, e = (l % LPR) * 16;
                    const i32x4 x = *reinterpret_cast<const i32x4*>(slot + L::OBOX + r * L::OROW + e);
                    if (r < len) *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(p.o + ((tok0 + r) * H + h) * V) + e) = x;
                }
            } else {
                constexpr int LPO = V * 4 / 16, RPO = 64 / LPO;
                char* ol = reinterpret_cast<char*>(a.ol + chw * (CH * V));
#pragma unroll
                for (int r0 = 0; r0 < CH / 2; r0 += RPO) {
                    const int r = rb + r0 + l / LPO, e = (l % LPO) * 16;
                    *reinterpret_cast<i32x4*>(ol + r * (V * 4) + e) = *reinterpret_cast<const i32x4*>(slot + L::OBOX + r * L::OROW + e);
                }
                constexpr int LPG = K * (int)sizeof(T) / 16, RPG = 64 / LPG;
                char* gw = reinterpret_cast<char*>(a.gw + chw * (CH * K));
#pragma unroll
                for (int r0 = 0; r0 < CH / 2; r0 += RPG) {
                    const int r = rb + r0 + l / LPG, e = (l % LPG) * 16;
                    *reinterpret_cast<i32x4*>(gw + r * (K * (int)sizeof(T)) + e) = *reinterpret_cast<const i32x4*>(slot + L::GBOX + r * L::GROW + e);
                }
            }
        }
    };

    // The wave's share of the chunk's inputs as loaded, four elements a lane (lane (g,c): token c, channels 16kt + 4g ..):
    // requested one chunk of this pair ahead, as soon as the registers are free, so that the round trip to HBM runs
    // behind the rest of the previous chunk.  Nothing is done to them at the load (a select or a conversion would wait
    // for the data).  With the HDLA parameterisation the sum over ALL channels of k^2 f is needed: the other half's k and
    // gk come along.
    Frag<T> nq[KH], nk[KH], na[2][KH], nb[2][KH], nv[VH], ndo[VH], ok_[KH];
    typename GkRaw<T, GKF32>::type ng[KH], og[KH];
    T nbeta;
    // first: the first own channel tile's operands (requested a chunk ahead); !first: everything else of the chunk
    // (requested when its turn begins: it arrives behind the work on the first tile).  More a chunk ahead would be more
    // registers held through the whole chunk than three waves per SIMD leave.
    auto request = [&](int t, bool first) __attribute__((always_inline)) {
        const int cid = REV ? s1 - 1 - t : s0 + t;
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        // uniform base of the chunk's first row + a 32-bit byte offset per lane, formed afresh in every call (see copy_out);
        // rows past the end alias the last valid row and are masked at use
        int cc = c, gg = g;
        asm volatile("" : "+v"(cc), "+v"(gg));
        const uint32_t row = (uint32_t)min(cc, max(len, 1) - 1);
        constexpr uint32_t ES = sizeof(T), GS = GKF32 ? 4 : 2;
        const uint32_t qe = row * (uint32_t)(H * K) + 4 * gg, ae = row * (uint32_t)(RANK * H * K) + 4 * gg;
        const uint32_t ve = row * (uint32_t)(H * V) + 4 * gg;
        const int64_t qb = (tok0 * H + h) * K, ab = (tok0 * RANK * H + h) * K, vb = (tok0 * H + h) * V;
        const char* gkp = reinterpret_cast<const char*>(p.gk) + qb * GS;
        if (!first) {
            if (!REV) {
#pragma unroll
                for (int j = 0; j < VH; ++j) nv[j] = ld_frag(at(p.v + vb, (ve + 16 * (vt0 + j)) * ES));
            }
            if (REV || CKPT) {
#pragma unroll
                for (int j = 0; j < VH; ++j) ndo[j] = ld_frag(at(p.dout + vb, (ve + 16 * (vt0 + j)) * ES));
            }
        }
        if (HD && first) nbeta = *at(p.beta + tok0 * H + h, row * (uint32_t)H * ES);
#pragma unroll
        for (int j = 0; j < KH; ++j) {
            const uint32_t ko = 16 * (kt0 + j), kx = 16 * (KH - kt0 + j);
            if (HD && first) {
                // the sum over all channels comes before everything else: k and gk of every tile a chunk ahead
                if (j > 0) {
                    ng[j] = GkRaw<T, GKF32>::load(gkp + (qe + ko) * GS);
                    nk[j] = ld_frag(at(p.k + qb, (qe + ko) * ES));
                }
                og[j] = GkRaw<T, GKF32>::load(gkp + (qe + kx) * GS);
                ok_[j] = ld_frag(at(p.k + qb, (qe + kx) * ES));
            }
            if ((j == 0) != first) continue;
            nq[j] = ld_frag(at(p.q + qb, (qe + ko) * ES));
            if (!(HD && j > 0)) {
                ng[j] = GkRaw<T, GKF32>::load(gkp + (qe + ko) * GS);
                nk[j] = ld_frag(at(p.k + qb, (qe + ko) * ES));
            }
            if (!HD) {
                na[0][j] = ld_frag(at(p.a + ab, (ae + ko) * ES));
                na[1][j] = ld_frag(at(p.a + ab, (ae + (uint32_t)(H * K) + ko) * ES));
                nb[0][j] = ld_frag(at(p.b + ab, (ae + ko) * ES));
                nb[1][j] = ld_frag(at(p.b + ab, (ae + (uint32_t)(H * K) + ko) * ES));
            }
        }
    };
    auto sel = [](Frag<T> f, bool ok) __attribute__((always_inline)) {
        Frag<T> r;
        r.v = ok ? f.v : zero_frag<T>().v;
        return r;
    };
    if (pp < nst) request(pp, true);

    int it = 0, prev_cid = -1;
    for (int t = pp; t < nst; t += FNP, ++it) {
        const int cid = REV ? s1 - 1 - t : s0 + t;
        const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
        const int len = (int)min((int64_t)CH, eos - tok0);
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        // What depends on the lane only (offsets into the slot, masks, the identity tile) is formed afresh for every chunk:
        // hoisted out of the loop it would be held in registers, or spilled, through all of it.
        asm volatile("" : "+v"(l));
        g = l >> 4;
        c = l & 15;
        {
            int so = pp * L::SLOT;
            asm volatile("" : "+s"(so));
            slot = smem + so;
            sP = reinterpret_cast<float*>(slot + L::SOLVE);
            sN = sP;
            sT = sP + 32 * FLDP;
            sPub = reinterpret_cast<T*>(sP);
        }
        const Frag<T> ident = ident_of<T>(g, c);
        const bool rowok = c < len;

        // ---- the slot: wait until the consumers have left the chunk it held ---------------------------------------------
        // (at the top, so that every tile can go to the slot as it is formed instead of being held in registers; the
        // consumers are through with the slot a step of theirs after this pair's last signal, long before this pair is
        // back here, unless they are what limits the kernel anyway)
        if (!wait_ge(f_consumed, VT * it, f_abort)) { if (l == 0) *a.err = FUSED_ABORTED + 1; return; }
        __builtin_amdgcn_sched_barrier(0);
        // The rows the consumers left in the outbox for that chunk go out first (the consumers write the outbox again
        // only after both signals at the end).
        if (it > 0) copy_out(prev_cid);
        prev_cid = cid;
        __builtin_amdgcn_sched_barrier(0);
        request(t, false);                                // the rest of this chunk's inputs, behind those stores
        __builtin_amdgcn_sched_barrier(0);
        // (ag^T waits in the slot where w will go: w = Tm ag is formed further down, when the inverse is there)
        T* const sWW = reinterpret_cast<T*>(slot + (REV ? SB.W : BF.W));

        // ---- own channel tiles: decays, parts of the score tiles, gated copies (prep.hip, phases A and C) -------------
        f32x4 aqk = zero4(), aqb[2] = {zero4(), zero4()}, aak[2] = {zero4(), zero4()};
        f32x4 aab[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
        f32x4 aqbT[2] = {zero4(), zero4()};
        float big = 0.f;                                  // see strong_decay()
        float beta_t = 0.f, s_t = 0.f;
        if (HD) {
            beta_t = rowok ? ld_elem(&nbeta) : 0.f;
#pragma unroll
            for (int j = 0; j < KH; ++j) {
                const f32x4 g4 = GkRaw<T, GKF32>::value(ng[j], rowok), gx = GkRaw<T, GKF32>::value(og[j], rowok);
                const f32x4 k4 = to_f32(sel(nk[j], rowok)), kx = to_f32(sel(ok_[j], rowok));
                const f32x4 kf = k4 * k4 * exp4<T>(g4) + kx * kx * exp4<T>(gx);
                s_t += kf[0] + kf[1] + kf[2] + kf[3];
            }
            s_t += __shfl_xor(s_t, 16);
            s_t += __shfl_xor(s_t, 32);
        }
        // the operands of channel tile j as the products take them: as loaded, or (HDLA parameterisation) formed from k,
        // gk, beta and s
        auto operands = [&](int j, f32x4 g4, Frag<T>& rq, Frag<T>& rk, Frag<T> (&ra)[2], Frag<T> (&rb)[2]) __attribute__((always_inline)) {
            rq = sel(nq[j], rowok);
            rk = sel(nk[j], rowok);
            if (HD) {
                const f32x4 kk = to_f32(rk), f4 = exp4<T>(g4);
                ra[0] = to_frag<T>(kk * (-beta_t));
                ra[1] = to_frag<T>(kk * ((beta_t * s_t - f4) * beta_t));
                rb[0] = to_frag<T>(f4 * kk);
                rb[1] = rk;
            } else {
                ra[0] = sel(na[0][j], rowok);
                ra[1] = sel(na[1][j], rowok);
                rb[0] = sel(nb[0][j], rowok);
                rb[1] = sel(nb[1][j], rowok);
            }
        };
        auto decays = [&](int j, f32x4& gi, f32x4& ge) __attribute__((always_inline)) {
            const f32x4 g4 = GkRaw<T, GKF32>::value(ng[j], rowok);
            gi = scan16_incl(g4);
            ge = gi - g4;
        };
#pragma unroll
        for (int j = 0; j < KH; ++j) {
            const f32x4 g4 = GkRaw<T, GKF32>::value(ng[j], rowok);
            Frag<T> rq, rk, ra[2], rb[2];
            operands(j, g4, rq, rk, ra, rb);
            const f32x4 gi = scan16_incl(g4), ge = gi - g4;
            const f32x4 m = bcast16<MID>(gi);
#pragma unroll
            for (int i = 0; i < 4; ++i) big = fmaxf(big, fmaxf(fabsf(gi[i] - m[i]), fabsf(ge[i] - m[i])));
            // One row-side operand at a time against the three inner-side ones, the scheduler kept from interleaving the
            // groups (each tile still gets its products in the order of the channel tiles): all six split operands
            // at once are more registers than three waves per SIMD leave.
            {
                const f32x4 ek = exp4<T>(m - gi);
                Split<T> kh, bh[2];
                split(to_f32(rk) * ek, kh);
                split(to_f32(rb[0]) * ek, bh[0]);
                split(to_f32(rb[1]) * ek, bh[1]);
                __builtin_amdgcn_sched_barrier(0);
                {
                    Split<T> qh;
                    split(to_f32(rq) * exp4<T>(gi - m) * scale, qh);
                    if (FWD) aqk = mm3(qh, kh, aqk);
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        if (!REV) aqb[s] = mm3(qh, bh[s], aqb[s]);
                        if (REV) aqbT[s] = mm3(bh[s], qh, aqbT[s]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                const f32x4 ea = exp4<T>(ge - m);
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    Split<T> ah;
                    split(to_f32(ra[r]) * ea, ah);
                    if (!REV) aak[r] = mm3(ah, kh, aak[r]);
                    aab[r][0] = mm3(ah, bh[0], aab[r][0]);
                    aab[r][1] = mm3(ah, bh[1], aab[r][1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            pin(rq); pin(rk); pin(ra[0]); pin(ra[1]); pin(rb[0]); pin(rb[1]);
            const f32x4 q4 = to_f32(rq), k4 = to_f32(rk);
            const f32x4 a0 = to_f32(ra[0]), a1 = to_f32(ra[1]), b0 = to_f32(rb[0]), b1 = to_f32(rb[1]);
            // the gated copies, while the operands are at hand: each tile goes to its half of the stored pair
            // (scheduling barriers: the products above, the copies below and the next tile are kept apart, or their
            // temporaries would all be live at once)
            __builtin_amdgcn_sched_barrier(0);
            const f32x4 gl = bcast16<CH - 1>(gi);
            const f32x4 egi = exp4<T>(gi), edn = exp4<T>(gl - gi);
            // e^{ge} of a token is e^{gi} of the token before it (1 for the first), e^{gl} is e^{gi} of the last token:
            // lane moves in place of two more rounds of exponentials
            f32x4 ege = dpp0<0x111>(egi);                 // row_shr:1 (lanes of one token group are a DPP row)
#pragma unroll
            for (int i = 0; i < 4; ++i) ege[i] = c == 0 ? 1.f : ege[i];
            const f32x4 egl = bcast16<CH - 1>(egi);
            st_pair(sWW + (0 * KT2 + half) * PAIR, j, transpose(to_frag<T>(a0 * ege), ident));
            st_pair(sWW + (1 * KT2 + half) * PAIR, j, transpose(to_frag<T>(a1 * ege), ident));
            const Frag<T> fqg = to_frag<T>(q4 * egi * scale);
            const Frag<T> fbg[2] = {to_frag<T>(b0 * edn), to_frag<T>(b1 * edn)};
            if (!REV) {
                st_pair(reinterpret_cast<T*>(slot + BF.KGT) + half * PAIR, j, transpose(to_frag<T>(k4 * edn), ident));
                st_pair(reinterpret_cast<T*>(slot + BF.BGT) + (0 * KT2 + half) * PAIR, j, transpose(fbg[0], ident));
                st_pair(reinterpret_cast<T*>(slot + BF.BGT) + (1 * KT2 + half) * PAIR, j, transpose(fbg[1], ident));
                st_pair(reinterpret_cast<T*>(slot + BF.QG) + half * PAIR, j, fqg);
            } else {
                // the reverse scan takes bg as it is and w transposed (the stand-alone kernel turns the stored tiles on
                // their way into LDS: the same values)
                st_pair(reinterpret_cast<T*>(slot + SB.BGT) + (0 * KT2 + half) * PAIR, j, fbg[0]);
                st_pair(reinterpret_cast<T*>(slot + SB.BGT) + (1 * KT2 + half) * PAIR, j, fbg[1]);
                st_pair(reinterpret_cast<T*>(slot + SB.QGT) + half * PAIR, j, transpose(fqg, ident));
            }
            if (c == 0) *reinterpret_cast<f32x4*>(slot + (REV ? SB.EGL : BF.EGL) + (16 * (kt0 + j) + 4 * g) * 4) = egl;
            __builtin_amdgcn_sched_barrier(0);
        }
        // Each wave decides for its own channels (the parts of the score tiles add up whichever way they were formed).
        // Where a channel decays too strongly for the single centre, what was accumulated above may hold infinities: it
        // is thrown away and the parts are formed again by passes whose exponents cannot overflow (see DecayPass).
        const bool strong = __any(big > SAFE_RANGE) != 0;  // the same answer on every lane of the wave
        if (strong) {
            aqk = zero4();
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                aqb[s] = zero4(); aak[s] = zero4(); aqbT[s] = zero4(); aab[0][s] = zero4(); aab[1][s] = zero4();
            }
#pragma unroll 1
            for (int ps = 0; ps < DecayPass::COUNT; ++ps) {
                const DecayPass dp(ps, c);
#pragma unroll
                for (int j = 0; j < KH; ++j) {
                    f32x4 gi, ge, eq, ek, ea;
                    decays(j, gi, ge);
                    dp.factors<T>(gi, ge, eq, ek, ea);
                    Frag<T> rq, rk, ra[2], rb[2];
                    operands(j, gi - ge, rq, rk, ra, rb);
                    pin(rk); pin(rq); pin(ra[0]); pin(ra[1]); pin(rb[0]); pin(rb[1]);
                    Split<T> qh, kh, bh[2];
                    split(to_f32(rk) * ek, kh);
                    split(to_f32(rq) * eq * scale, qh);
                    if (FWD) aqk = mm3(qh, kh, aqk);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        split(to_f32(rb[s]) * ek, bh[s]);
                        if (!REV) aqb[s] = mm3(qh, bh[s], aqb[s]);
                        if (REV) aqbT[s] = mm3(bh[s], qh, aqbT[s]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
#pragma unroll
                    for (int r = 0; r < 2; ++r) {
                        Split<T> ah;
                        split(to_f32(ra[r]) * ea, ah);
                        if (!REV) aak[r] = mm3(ah, kh, aak[r]);
                        aab[r][0] = mm3(ah, bh[0], aab[r][0]);
                        aab[r][1] = mm3(ah, bh[1], aab[r][1]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        // the first tile's inputs are used up: the next chunk's may come
        __builtin_amdgcn_sched_barrier(0);
        if (t + FNP < nst) request(t + FNP, true);
        __builtin_amdgcn_sched_barrier(0);

        // ---- the other wave's parts travel to the lead ------------------------------------------------------------------
        // tile order in the scratch: A_ab (4), then A_ak (2; the reverse kernel: A_qb^T), A_qb (2), A_qk: as many as the mode forms
        constexpr int NPART = REV ? 6 : FWD ? 9 : 8;    // A_ab, (A_ak), A_qb or its transpose, (A_qk)
        if (!lead) {
            f32x4* const tiles[9] = {&aab[0][0], &aab[0][1], &aab[1][0], &aab[1][1], REV ? &aqbT[0] : &aak[0], REV ? &aqbT[1] : &aak[1],
                                     &aqb[0], &aqb[1], &aqk};
#pragma unroll
            for (int i = 0; i < NPART; ++i) *reinterpret_cast<f32x4*>(sP + (i * 64 + l) * 4) = *tiles[i];
            if (l == 0) *f_strong = strong;
            signal_set(f_part, it + 1);
        }

        Frag<T> vT[VH];
        if (!REV) {
#pragma unroll
            for (int j = 0; j < VH; ++j) {
                vT[j] = transpose(sel(nv[j], rowok), ident);
                st_frag(reinterpret_cast<T*>(slot + L::VTT) + (vt0 + j) * TILE + 4 * l, vT[j]);
            }
        }
        if (REV || CKPT) {
            // rows past the end of a ragged chunk were taken as zeros
#pragma unroll
            for (int j = 0; j < VH; ++j) st_frag(reinterpret_cast<T*>(slot + L::DOT) + (vt0 + j) * TILE + 4 * l, transpose(sel(ndo[j], rowok), ident));
        }

        // ---- the lead: whole score tiles, (I - A_ab)^-1 by forward substitution (prep.hip, phase B) ---------------------
        Frag<T> tm[2][2], aakf[2];
        if (lead) {
            if (!wait_ge(f_part, it + 1, f_abort)) { if (l == 0) *a.err = FUSED_ABORTED + 1; return; }
            f32x4* const tiles[9] = {&aab[0][0], &aab[0][1], &aab[1][0], &aab[1][1], REV ? &aqbT[0] : &aak[0], REV ? &aqbT[1] : &aak[1],
                                     &aqb[0], &aqb[1], &aqk};
            // the lower channel tiles' part first, as a single wave adds them
#pragma unroll
            for (int i = 0; i < NPART; ++i) {
                const f32x4 o = *reinterpret_cast<const f32x4*>(sP + (i * 64 + l) * 4);
                *tiles[i] = half == 0 ? *tiles[i] + o : o + *tiles[i];
            }
            if (CKPT && l == 0) p.ws.STRONG[chw] = (strong || *f_strong != 0) ? 1 : 0;
            // causal masks: lane (g,c) reg i is entry (row c, inner 4g+i)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = 4 * g + i;
                const bool le = j <= c, lt = j < c, tle = c <= j;
                if (!le) { aqk[i] = 0.f; aqb[0][i] = 0.f; aqb[1][i] = 0.f; }
                if (!lt) { aak[0][i] = 0.f; aak[1][i] = 0.f; aab[0][0][i] = 0.f; aab[0][1][i] = 0.f; aab[1][0][i] = 0.f; aab[1][1][i] = 0.f; }
                if (!tle) { aqbT[0][i] = 0.f; aqbT[1][i] = 0.f; }
            }
            if (!REV) {
                if (FWD) st_frag(reinterpret_cast<T*>(slot + BF.AQK) + 4 * l, to_frag<T>(aqk));
                st_pair2(reinterpret_cast<T*>(slot + BF.AQB), to_frag<T>(aqb[0]), to_frag<T>(aqb[1]));
            } else {
                st_pair2(reinterpret_cast<T*>(slot + SB.AQBT), to_frag<T>(aqbT[0]), to_frag<T>(aqbT[1]));
            }
            aakf[0] = to_frag<T>(aak[0]);
            aakf[1] = to_frag<T>(aak[1]);
            // (all of the other wave's parts have been read: the scratch may be written)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    *reinterpret_cast<f32x4*>(&sN[(16 * r + c) * FLDP + 16 * s + 4 * g]) = aab[r][s];
            __builtin_amdgcn_sched_barrier(0);
            // The system in token halves, L = tokens 0..7 and H = 8..15 (both ranks: 16 rows each):
            //   (I - A)^-1 = [[T_LL, 0], [T_HL, T_HH]],  T_LL = (I - A_LL)^-1,  T_HH = (I - A_HH)^-1,  T_HL = T_HH A_HL T_LL.
            // The two diagonal blocks are independent eight-step substitutions that run side by side on the lanes (a
            // quarter of the dependent multiply-adds of one sixteen-step substitution); the block below the diagonal is
            // two 16 x 16 x 16 products, in split operands like the score products (the error of fp32 products).
            {
                int lb = l;                               // formed afresh per chunk (see copy_out)
                asm volatile("" : "+v"(lb));
                // lane: rank of the rows r, token half hf, column (rank sc, token jc of the same half)
                const int r = lb >> 5, hf = (lb >> 4) & 1, sc = (lb >> 3) & 1, jc = lb & 7;
                const int col = 16 * sc + 8 * hf + jc;
                float x[8], y[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float* nrow = &sN[(16 * r + 8 * hf + i) * FLDP + 8 * hf];
                    float acc0 = (sc == r && jc == i) ? 1.f : 0.f, acc1 = 0.f;
#pragma unroll
                    for (int j4 = 0; j4 < (i + 3) / 4; ++j4) {
                        const f32x4 co = *reinterpret_cast<const f32x4*>(nrow + 16 * r + 4 * j4);
                        const f32x4 cx = *reinterpret_cast<const f32x4*>(nrow + 16 * (1 - r) + 4 * j4);
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {
                            const int j = 4 * j4 + jj;
                            if (j < i) { acc0 = fmaf(co[jj], x[j], acc0); acc1 = fmaf(cx[jj], y[j], acc1); }
                        }
                    }
                    x[i] = acc0 + acc1;
                    y[i] = xor32(x[i]);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    sT[(16 * r + 8 * hf + i) * FLDP + col] = x[i];
                    // the block above the diagonal (rows of L, columns of H) is zero: the lanes of L write it
                    if (hf == 0) sT[(16 * r + i) * FLDP + col + 8] = 0.f;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                // 16 x 16 matrices in (rank, token of the half) order: row c = 8 rank + token, inner 4g .. 4g+3 likewise
                const int rr = c >> 3, ii = c & 7, ss = g >> 1, j0 = 4 * (g & 1);
                const f32x4 ahl = *reinterpret_cast<const f32x4*>(&sN[(16 * rr + 8 + ii) * FLDP + 16 * ss + j0]);
                const f32x4 thh = *reinterpret_cast<const f32x4*>(&sT[(16 * rr + 8 + ii) * FLDP + 16 * ss + 8 + j0]);
                f32x4 tllT;                               // T_LL^T: row c is column c of T_LL
#pragma unroll
                for (int e = 0; e < 4; ++e) tllT[e] = sT[(16 * ss + j0 + e) * FLDP + 16 * rr + ii];
                Split<T> pa, pb;
                split(tllT, pa);
                split(ahl, pb);
                const f32x4 xT = mm3(pa, pb, zero4());    // (A_HL T_LL)^T = T_LL^T A_HL^T
                split(thh, pa);
                split(xT, pb);
                const f32x4 thl = mm3(pa, pb, zero4());   // T_HH (A_HL T_LL)
                *reinterpret_cast<f32x4*>(&sT[(16 * rr + 8 + ii) * FLDP + 16 * ss + j0]) = thl;
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
                    tm[s][s2] = to_frag<T>(*reinterpret_cast<const f32x4*>(&sT[(16 * s + c) * FLDP + 16 * s2 + 4 * g]));
            // for the other wave: the inverse's four blocks and A_ak as operand tiles (in A_ab's bytes, which are used up)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 2; ++s) st_pair2(sPub + s * PAIR, tm[s][0], tm[s][1]);
            st_pair2(sPub + 2 * PAIR, aakf[0], aakf[1]);
            if (CKPT) {
                // What the checkpoint pass leaves in the workspace for chunk_grad ((I - A_ab)^-1 here, u and where needed w
                // below) goes there from the consumers, which have no loads to wait for: a store issued here would stand
                // behind the next chunk's loads in this wave's in-order memory counter.
                T* tmw = reinterpret_cast<T*>(slot + L::TMB);
#pragma unroll
                for (int s = 0; s < 2; ++s) st_pair2(tmw + s * PAIR, transpose(tm[s][0], ident), transpose(tm[s][1], ident));
            }
            signal_set(f_inv, it + 1);
        } else {
            if (!wait_ge(f_inv, it + 1, f_abort)) { if (l == 0) *a.err = FUSED_ABORTED + 1; return; }
#pragma unroll
            for (int s = 0; s < 2; ++s) ld_pair(sPub + s * PAIR, tm[s][0], tm[s][1]);
            ld_pair(sPub + 2 * PAIR, aakf[0], aakf[1]);
        }
        // ---- w = Tm ag for the own channel tiles, in place of ag^T -------------------------------------------------------
        {
            Frag<T> agT[2][2], fw[2][2];
            ld_pair(sWW + (0 * KT2 + half) * PAIR, agT[0][0], agT[0][1]);
            ld_pair(sWW + (1 * KT2 + half) * PAIR, agT[1][0], agT[1][1]);
#pragma unroll
            for (int e = 0; e < 2; ++e)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    f32x4 w = mm(tm[s][0], agT[0][e], zero4());
                    w = mm(tm[s][1], agT[1][e], w);
                    fw[s][e] = to_frag<T>(w);
                }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if (!REV) st_pair2(sWW + (s * KT2 + half) * PAIR, fw[s][0], fw[s][1]);
                else st_pair2(sWW + (s * KT2 + half) * PAIR, transpose(fw[s][0], ident), transpose(fw[s][1], ident));
            }
        }
        // ---- u = Tm (A_ak v) for the own value tiles, transposed (prep.hip, phase D) ------------------------------------
        if (!REV) {
#pragma unroll
            for (int j = 0; j < VH; ++j) {
                const Frag<T> mT[2] = {to_frag<T>(mm(vT[j], aakf[0], zero4())), to_frag<T>(mm(vT[j], aakf[1], zero4()))};
                Frag<T> fu[2];
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    f32x4 uT = mm(mT[0], tm[s][0], zero4());
                    uT = mm(mT[1], tm[s][1], uT);
                    fu[s] = to_frag<T>(uT);
                }
                st_pair2(reinterpret_cast<T*>(slot + L::UT) + (vt0 + j) * PAIR, fu[0], fu[1]);
            }
        }
        signal_add(f_ready);
    }
    // the last chunk's rows
    if (FWD && it > 0) {
        if (!wait_ge(f_consumed, VT * it, f_abort)) { if (l == 0) *a.err = FUSED_ABORTED + 1; return; }
        copy_out(prev_cid);
    }
}

// ---- consumers, forward direction ----------------------------------------------------------------------------------
// Fragment-order records in the workspace (256 fp32 per tile, lane l owns elements 4l..4l+3), per (sequence, head,
// segment):
//   sloc  [V/16][K/16] tiles  F(S^T): the state leaving the segment (started from h0 / the given boundary in segment
//                             0 and in checkpoint mode, from zero otherwise)
//   mseg  [K/16][K/16] tiles  the segment's transition M (segments > 0).  Forward pass: tile (kt, k't) = F(M block),
//                             rows k, inner k'; checkpoint mode: the transposed block, rows k', inner k
//   rseg  [V/16][K/16] tiles  F(R^T), R = sum_t G_t^T do_t (checkpoint mode, segments > 0)
//   sin   [V/16][K/16] tiles  F(S_in^T): the state entering the segment (segments > 0)
// W_GLOBAL: chunk_grad reads w from the workspace where it cannot rebuild it (chunk_grad_body.inc: REBUILD_W)
template <typename T, int K, int V, int MODE, bool W_GLOBAL>
__device__ __forceinline__ void fused_consumer_fwd(const FusedArgs<T>& a, char* smem, int n, int h, int seg, int s0, int s1, int wv) {
    typedef FusedLds<T, K, V, MODE> L;
    constexpr bool CKPT = MODE == FUSED_CKPT, FWD = MODE == FUSED_FWD;
    constexpr int KT = K / 16, VT = V / 16, KT2 = KT / 2;
    static_assert(KT == VT, "consumer j owns column block j of the state and of the transition matrix");
    constexpr BlkF BF = L::BF;
    const ChunkArgs<T>& p = a.c;
    int* const flags = reinterpret_cast<int*>(smem + L::FLAGS);
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H, vt = wv;
    const int nst = s1 - s0;
    const bool pblk = seg > 0;                            // uniform over the workgroup
    const int64_t rec = ((int64_t)n * H + h) * a.nseg + seg;
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;

    // state block: lane (g,c) reg i of tile kt = S[16kt + 4g + i][16vt + c]; likewise M with column 16vt + c
    f32x4 S[KT], M[KT], R[VT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        S[kt] = zero4();
#pragma unroll
        for (int i = 0; i < 4; ++i) M[kt][i] = (16 * kt + 4 * g + i == 16 * vt + c) ? 1.f : 0.f;
    }
#pragma unroll
    for (int j = 0; j < VT; ++j) R[j] = zero4();
    if (seg == 0) {
        if (p.h0) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) S[kt][i] = p.h0[soff + (int64_t)(16 * kt + 4 * g + i) * V];
        }
    } else if (CKPT) {
        const float* sin = a.sin + rec * (K * V);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) S[kt] = *reinterpret_cast<const f32x4*>(sin + (vt * KT + kt) * TILE + 4 * l);
    }
    const Frag<T> ident = ident_frag<T>();

    for (int t = 0; t < nst; ++t) {
        const int pp = t & (FNP - 1), it = t / FNP;
        if (!wait_ge(&flags[pp], 2 * (it + 1), &flags[8])) { if (l == 0) *a.err = FUSED_ABORTED + 2; return; }
        const char* slot = smem + pp * L::SLOT;
        const int cid = s0 + t;
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        const T* sW = reinterpret_cast<const T*>(slot + BF.W);
        const T* sBGT = reinterpret_cast<const T*>(slot + BF.BGT);
        const T* sKGT = reinterpret_cast<const T*>(slot + BF.KGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + BF.EGL);
        Frag<T> w[2][KT], qg[KT], aqb[2], aqk, kgt[KT], bgt[2][KT], ut[2], vtt;
        f32x4 egl[KT];
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            ld_pair(sW + (0 * KT2 + kp) * PAIR, w[0][2 * kp], w[0][2 * kp + 1]);
            ld_pair(sW + (1 * KT2 + kp) * PAIR, w[1][2 * kp], w[1][2 * kp + 1]);
        }
        ld_pair(reinterpret_cast<const T*>(slot + L::UT) + wv * PAIR, ut[0], ut[1]);
        vtt = ld_tile(reinterpret_cast<const T*>(slot + L::VTT) + wv * TILE);
        if (FWD || pblk) {
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) ld_pair(reinterpret_cast<const T*>(slot + BF.QG) + kp * PAIR, qg[2 * kp], qg[2 * kp + 1]);
            ld_pair(reinterpret_cast<const T*>(slot + BF.AQB), aqb[0], aqb[1]);
        }
        if (FWD) aqk = ld_tile(reinterpret_cast<const T*>(slot + BF.AQK));
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            ld_pair(sKGT + kp * PAIR, kgt[2 * kp], kgt[2 * kp + 1]);
            ld_pair(sBGT + (0 * KT2 + kp) * PAIR, bgt[0][2 * kp], bgt[0][2 * kp + 1]);
            ld_pair(sBGT + (1 * KT2 + kp) * PAIR, bgt[1][2 * kp], bgt[1][2 * kp + 1]);
            egl[2 * kp] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp) + 4 * g);
            egl[2 * kp + 1] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp + 1) + 4 * g);
        }

        // ---- the state's column block: the stand-alone scan's step (scan_impl.cuh), operation for operation ---------
        Frag<T> sb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) sb[kt] = to_frag<T>(S[kt]);
        f32x4 vn[2] = {to_f32(ut[0]), to_f32(ut[1])};
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            vn[0] = mm(sb[kt], w[0][kt], vn[0]);
            vn[1] = mm(sb[kt], w[1][kt], vn[1]);
        }
        f32x4 o = zero4();
        if (FWD) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) o = mm(qg[kt], sb[kt], o);
            o = mm(aqk, vtt, o);
        }
        const Frag<T> vnb[2] = {to_frag<T>(vn[0]), to_frag<T>(vn[1])};
        if (CKPT) {
            T* hc = p.ws.HC + chw * (K * V) + vt * PAIR;
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) st_pair2(hc + kp * (VT * PAIR), sb[2 * kp], sb[2 * kp + 1]);
            // the producer's results that chunk_grad reads: between the waves the two tile pairs of (I - A_ab)^-1 and,
            // where chunk_grad does not rebuild them, this wave's tiles of u and the 2 KT/2 pairs of w
            if (W_GLOBAL) st_pair2(p.ws.UT + (chw * VT + vt) * PAIR, ut[0], ut[1]);
            if (wv < 2) {
                Frag<T> t0, t1;
                ld_pair(reinterpret_cast<const T*>(slot + L::TMB) + wv * PAIR, t0, t1);
                st_pair2(p.ws.TM + chw * 1024 + wv * PAIR, t0, t1);
            }
            if (W_GLOBAL) {
                static_assert(!W_GLOBAL || 2 * KT2 == VT, "one pair of w per consumer");
                T* wg = p.ws.W + chw * (p.ws.sa_stride / (int)sizeof(T));
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int kp = 0; kp < KT2; ++kp)
                        if (wv == s * KT2 + kp) st_pair2(wg + (s * KT2 + kp) * PAIR, w[s][2 * kp], w[s][2 * kp + 1]);
            }
        }
        if (FWD) {
            o = mm(aqb[0], vnb[0], o);
            o = mm(aqb[1], vnb[1], o);
            char* ob = smem + pp * L::SLOT + L::OBOX + c * L::OROW;
            if (seg == 0) st_frag(reinterpret_cast<T*>(ob) + 16 * wv + 4 * g, to_frag<T>(o));
            else *reinterpret_cast<f32x4*>(ob + (16 * wv + 4 * g) * 4) = o;
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 x = S[kt] * egl[kt];
            x = mm(vtt, kgt[kt], x);
            x = mm(vnb[0], bgt[0][kt], x);
            x = mm(vnb[1], bgt[1][kt], x);
            S[kt] = x;
        }
        // ---- the transition matrix's column block: the same update without the chunk's own input --------------------
        if (pblk) {
            Frag<T> mb[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) mb[kt] = to_frag<T>(M[kt]);
            f32x4 vp[2] = {zero4(), zero4()};
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                vp[0] = mm(mb[kt], w[0][kt], vp[0]);
                vp[1] = mm(mb[kt], w[1][kt], vp[1]);
            }
            f32x4 G = zero4();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) G = mm(qg[kt], mb[kt], G);
            const Frag<T> vpb[2] = {to_frag<T>(vp[0]), to_frag<T>(vp[1])};
            G = mm(aqb[0], vpb[0], G);
            G = mm(aqb[1], vpb[1], G);
            const Frag<T> Gf = to_frag<T>(G);             // rows token, inner k' (the block's columns)
            if (FWD) st_frag(reinterpret_cast<T*>(smem + pp * L::SLOT + L::GBOX + c * L::GROW) + 16 * wv + 4 * g, Gf);
            if (CKPT) {
                // R[k'][v] += sum_tok G[tok][k'] do[tok][v]
                const Frag<T> GT = transpose(Gf, ident);
#pragma unroll
                for (int j = 0; j < VT; ++j) R[j] = mm(GT, ld_tile(reinterpret_cast<const T*>(slot + L::DOT) + j * TILE), R[j]);
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                f32x4 x = M[kt] * egl[kt];
                x = mm(vpb[0], bgt[0][kt], x);
                x = mm(vpb[1], bgt[1][kt], x);
                M[kt] = x;
            }
        }
        signal_add(&flags[4 + pp]);
    }

    // ---- what the segment leaves behind ------------------------------------------------------------------------------
    if (a.nseg == 1) {
        if (p.ht && !CKPT) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
        }
        return;
    }
    if (!CKPT) {
        float* sloc = a.sloc + rec * (K * V);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<f32x4*>(sloc + (vt * KT + kt) * TILE + 4 * l) = S[kt];
    }
    if (pblk) {
        float* mseg = a.mseg + rec * (K * K);
        const Frag<float> identf = ident_frag<float>();
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            Frag<float> f;
            f.v = M[kt];
            if (!CKPT) f = transpose(f, identf);          // exact: fp32 products with ones and zeros
            *reinterpret_cast<f32x4*>(mseg + (kt * KT + wv) * TILE + 4 * l) = f.v;
        }
        if (CKPT) {
            float* rseg = a.rseg + rec * (K * V);
#pragma unroll
            for (int j = 0; j < VT; ++j) {
                Frag<float> f;
                f.v = R[j];
                f = transpose(f, identf);
                *reinterpret_cast<f32x4*>(rseg + (j * KT + wv) * TILE + 4 * l) = f.v;
            }
        }
    }
}

// ---- consumers, reverse direction ------------------------------------------------------------------------------------
template <typename T, int K, int V>
__device__ __forceinline__ void fused_consumer_rev(const FusedArgs<T>& a, char* smem, int n, int h, int seg, int s0, int s1, int wv) {
    typedef FusedLds<T, K, V, FUSED_REV> L;
    constexpr int KT = K / 16, VT = V / 16, KT2 = KT / 2;
    constexpr SlotB B = L::SB;
    const ChunkArgs<T>& p = a.c;
    int* const flags = reinterpret_cast<int*>(smem + L::FLAGS);
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H, vt = wv;
    const int nst = s1 - s0;
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;

    f32x4 dS[KT];   // lane (g,c) reg i of tile kt = dS[16kt + 4g + i][16vt + c]
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) dS[kt] = zero4();
    if (p.dht) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) dS[kt][i] = p.dht[soff + (int64_t)(16 * kt + 4 * g + i) * V];
    }
    // The gradient entering this segment from the right: through the later segments, last one first,
    //   dS <- M_s^T dS + R_s   (as fragments: X^T <- X^T Q^T + A^T, tile (in, out) of the record at index in * KT + out).
    // Nothing waits for the producers here, so only the chain's own latency counts: the records of up to CHAIN_STAGE
    // segments are requested at once, a quarter of each transition record by each of the four consumer waves, which
    // share them through LDS as split operands; the consumers meet at two counters of their own (the producers are
    // at work meanwhile, so no workgroup barrier).
    {
        static_assert(VT == 4 && KT == 4, "a quarter of a record per consumer wave");
        constexpr int NQ = KT * KT / 4, STG = L::CHAIN_STAGE;
        // (one lane address for the whole area, opaque to the compiler: the area lies beyond the reach of an LDS
        // instruction's immediate offset from zero, and a register per tile address would not fit)
        int sMo = L::CHAIN + 4 * l * (int)sizeof(T);
        asm volatile("" : "+v"(sMo));
        T* const sM = reinterpret_cast<T*>(smem + sMo);
        const int64_t rec0 = ((int64_t)n * H + h) * a.nseg;
        int batch = 0, s = a.nseg - 1;
        while (s > seg) {
            int step[STG], ns = 0, q0, q1;
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                step[b] = 0;
                while (s > seg) {
                    seg_range(p.st, n, a.nseg, s, q0, q1);
                    if (q1 > q0) break;
                    --s;
                }
                if (s > seg) { step[b] = s--; ns = b + 1; }
            }
            f32x4 mq[STG][NQ], add[STG][KT];
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                if (b < ns) {
                    const float* mrec = a.mseg + (rec0 + step[b]) * (K * K) + wv * NQ * TILE + 4 * l;
#pragma unroll
                    for (int i = 0; i < NQ; ++i) mq[b][i] = *reinterpret_cast<const f32x4*>(mrec + i * TILE);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                if (b < ns) {
                    const float* rrec = a.rseg + (rec0 + step[b]) * (K * V) + vt * KT * TILE + 4 * l;
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) add[b][kt] = *reinterpret_cast<const f32x4*>(rrec + kt * TILE);
                }
            }
            // every consumer has read the previous round's records out of LDS
            if (batch > 0 && !wait_ge(&flags[25], VT * batch, &flags[8])) { if (l == 0) *a.err = FUSED_ABORTED + 3; return; }
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                if (b < ns) {
#pragma unroll
                    for (int i = 0; i < NQ; ++i) {
                        Split<T> q;
                        split(mq[b][i], q);
                        st_frag(sM + ((b * 2 + 0) * KT * KT + wv * NQ + i) * TILE, q.hi);
                        st_frag(sM + ((b * 2 + 1) * KT * KT + wv * NQ + i) * TILE, q.lo);
                    }
                }
            }
            signal_add(&flags[24]);
            if (!wait_ge(&flags[24], VT * (batch + 1), &flags[8])) { if (l == 0) *a.err = FUSED_ABORTED + 3; return; }
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                if (b < ns) {
                    Split<T> xs[KT];
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) split(dS[kt], xs[kt]);
#pragma unroll
                    for (int ko = 0; ko < KT; ++ko) {
                        f32x4 acc = add[b][ko];
#pragma unroll
                        for (int ki = 0; ki < KT; ++ki) {
                            Split<T> q;
                            q.hi = ld_frag(sM + ((b * 2 + 0) * KT * KT + ki * KT + ko) * TILE);
                            q.lo = ld_frag(sM + ((b * 2 + 1) * KT * KT + ki * KT + ko) * TILE);
                            acc = mm3(xs[ki], q, acc);
                        }
                        dS[ko] = acc;
                    }
                }
            }
            signal_add(&flags[25]);
            ++batch;
        }
    }

    for (int t = 0; t < nst; ++t) {
        const int pp = t & (FNP - 1), it = t / FNP;
        if (!wait_ge(&flags[pp], 2 * (it + 1), &flags[8])) { if (l == 0) *a.err = FUSED_ABORTED + 3; return; }
        const char* slot = smem + pp * L::SLOT;
        const int cid = s1 - 1 - t;
        const int64_t chw = (int64_t)h * p.st.nch + cid;
        const T* sWT = reinterpret_cast<const T*>(slot + B.W);
        const T* sBG = reinterpret_cast<const T*>(slot + B.BGT);
        const T* sQGT = reinterpret_cast<const T*>(slot + B.QGT);
        const float* sEGL = reinterpret_cast<const float*>(slot + B.EGL);
        Frag<T> aq[2], bg[2][KT], qgt[KT], wt[2][KT];
        f32x4 egl[KT];
        ld_pair(reinterpret_cast<const T*>(slot + B.AQBT), aq[0], aq[1]);
        const Frag<T> doT = ld_tile(reinterpret_cast<const T*>(slot + L::DOT) + wv * TILE);
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) {
            ld_pair(sBG + (0 * KT2 + kp) * PAIR, bg[0][2 * kp], bg[0][2 * kp + 1]);
            ld_pair(sBG + (1 * KT2 + kp) * PAIR, bg[1][2 * kp], bg[1][2 * kp + 1]);
            ld_pair(sQGT + kp * PAIR, qgt[2 * kp], qgt[2 * kp + 1]);
            ld_pair(sWT + (0 * KT2 + kp) * PAIR, wt[0][2 * kp], wt[0][2 * kp + 1]);
            ld_pair(sWT + (1 * KT2 + kp) * PAIR, wt[1][2 * kp], wt[1][2 * kp + 1]);
            egl[2 * kp] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp) + 4 * g);
            egl[2 * kp + 1] = *reinterpret_cast<const f32x4*>(sEGL + 16 * (2 * kp + 1) + 4 * g);
        }
        // the stand-alone reverse scan's step (scan_impl.cuh), operation for operation
        Frag<T> dsb[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) dsb[kt] = to_frag<T>(dS[kt]);
        f32x4 dvn[2];
        dvn[0] = mm(doT, aq[0], zero4());
        dvn[1] = mm(doT, aq[1], zero4());
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            dvn[0] = mm(dsb[kt], bg[0][kt], dvn[0]);
            dvn[1] = mm(dsb[kt], bg[1][kt], dvn[1]);
        }
        const Frag<T> dvb[2] = {to_frag<T>(dvn[0]), to_frag<T>(dvn[1])};
        T* dhc = p.ws.DHC + chw * (K * V) + vt * PAIR;
        T* dvp = p.ws.DVN + chw * (2 * CH * V) + vt * PAIR;
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) st_pair2(dhc + kp * (VT * PAIR), dsb[2 * kp], dsb[2 * kp + 1]);
        st_pair2(dvp, dvb[0], dvb[1]);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            f32x4 x = dS[kt] * egl[kt];
            x = mm(doT, qgt[kt], x);
            x = mm(dvb[0], wt[0][kt], x);
            x = mm(dvb[1], wt[1][kt], x);
            dS[kt] = x;
        }
        signal_add(&flags[4 + pp]);
    }
    if (seg == 0 && p.dh0) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.dh0[soff + (int64_t)(16 * kt + 4 * g + i) * V] = dS[kt][i];
    }
}

// ---- the kernel ------------------------------------------------------------------------------------------------------
// grid = (H, nseg, N); block = 64 (V/16 + 2 FNP): waves 0 .. V/16-1 consume, the rest produce in pairs
template <typename T, bool GKF32, int K, int V, int MODE, bool HD>
__global__ __launch_bounds__(64 * (V / 16 + 2 * FNP)) void fused_kernel(FusedArgs<T> a) {
    typedef FusedLds<T, K, V, MODE> L;
    __shared__ __attribute__((aligned(16))) char smem[L::BYTES];
    const int h = blockIdx.x, seg = blockIdx.y;
    const int n = a.c.st.cu ? a.c.st.order[blockIdx.z] : (int)blockIdx.z;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int s0, s1;
    seg_range(a.c.st, n, a.nseg, seg, s0, s1);
    // an empty segment leaves nothing behind (whoever chains the segments skips it), except that the first one of an
    // empty sequence still passes the state through
    if (s1 <= s0 && seg > 0) return;
    if (threadIdx.x < 32) reinterpret_cast<int*>(smem + L::FLAGS)[threadIdx.x] = 0;
    __syncthreads();
    if (wv < V / 16) {
        if constexpr (MODE == FUSED_REV) fused_consumer_rev<T, K, V>(a, smem, n, h, seg, s0, s1, wv);
        else fused_consumer_fwd<T, K, V, MODE, MODE == FUSED_CKPT && (HD || GKF32)>(a, smem, n, h, seg, s0, s1, wv);
    } else {
        fused_producer<T, GKF32, K, V, MODE, HD>(a, smem, n, h, seg, s0, s1, (wv - V / 16) >> 1, (wv - V / 16) & 1);
    }
}

// ---- forward pass, second kernel: the true entering states, and their part of the output ----------------------------
// grid = (H, nseg * FIXUP_PARTS, N), 256 threads.  blockIdx.y / FIXUP_PARTS = s in 1 .. nseg-1: segment s (chain the
// records of segments 0 .. s-1 into S_in(s), keep it as the boundary record, add G S_in(s) to the segment's local
// outputs); 0: the final state (all segments chained).  The kernel is a chain of dependent steps between two launches,
// so everything is arranged for its latency: all loads that do not depend on the chain are issued at the start (the
// first chunks' operands, the records of up to FIXUP_STAGE chain steps); the transition records, which every wave needs
// whole, are loaded a quarter by each wave and shared through LDS as split operands; wave j chains column block j of
// the state (the blocks are independent); FIXUP_PARTS workgroups share the chunks of a segment, each repeating the
// chain, so that a workgroup's share of the chunks is in flight from the start as well.
constexpr int FIXUP_PARTS = 2;                            // workgroups that share one segment's chunks (measured: 1, 2, 4 -> 17.1, 16.8, 18.8 us)
constexpr int FIXUP_STAGE = 3;                            // chain steps whose records are in LDS at a time
template <typename T, int K, int V>
__global__ __launch_bounds__(256) void fixup_kernel(FusedArgs<T> a) {
    constexpr int KT = K / 16, VT = V / 16, NB = 2, NQ = KT * KT / 4;
    static_assert(VT == 4 && KT == 4 && sizeof(T) == 2, "one column block per wave, a quarter of a transition record per wave");
    constexpr int OROW = V * (int)sizeof(T) + 16;
    __shared__ __attribute__((aligned(16))) char stage[4][CH * OROW];
    __shared__ __attribute__((aligned(16))) T sS[VT * KT * TILE];          // S_in as operand tiles [vt][kt]
    __shared__ __attribute__((aligned(16))) T sM[FIXUP_STAGE][2][KT * KT * TILE];   // transition records, hi and lo halves
    const ChunkArgs<T>& p = a.c;
    const int h = blockIdx.x;
    const int n = p.st.cu ? p.st.order[blockIdx.z] : (int)blockIdx.z;
    const int ty = (int)blockIdx.y / FIXUP_PARTS, part = (int)blockIdx.y % FIXUP_PARTS;
    const int target = ty == 0 ? a.nseg : ty;                            // chain segments 0 .. target-1
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H, vt = wv;
    int s0 = 0, s1 = 0;
    if (target < a.nseg) {
        seg_range(p.st, n, a.nseg, target, s0, s1);
        // this workgroup's share of the segment's chunks
        const int per = (s1 - s0 + FIXUP_PARTS - 1) / FIXUP_PARTS;
        s0 = min(s0 + part * per, s1);
        s1 = min(s0 + per, s1);
        if (s1 <= s0 || (part > 0 && !a.gw)) return;
    } else if (!p.ht || part > 0) return;
    const int64_t rec0 = ((int64_t)n * H + h) * a.nseg;
    const int64_t soff = ((int64_t)n * H + h) * K * V + 16 * vt + c;

    int c0, c1;
    seq_chunks(p.st, n, c0, c1);
    int64_t bos, eos;
    seq_bounds(p.st, n, bos, eos);
    Frag<T> G[NB][KT];
    f32x4 OLr[NB][VT];
    auto request = [&](int first) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int cid = min(first + 4 * b, s1 - 1);   // past the end: the last chunk again, never used
            const int64_t chw = (int64_t)h * p.st.nch + cid;
            const T* gw = a.gw + chw * (CH * K) + c * K + 4 * g;
            const float* ol = a.ol + chw * (CH * V) + c * V + 4 * g;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) G[b][kt] = ld_frag(gw + 16 * kt);
#pragma unroll
            for (int j = 0; j < VT; ++j) OLr[b][j] = *reinterpret_cast<const f32x4*>(ol + 16 * j);
        }
    };
    const bool outputs = target < a.nseg && a.gw != nullptr;
    if (outputs) request(s0 + wv);

    // S[kt]: lane (g,c) reg i = S[16kt + 4g + i][16vt + c].  Segment 0 ran from the initial state itself; only where it
    // is empty does the chain start from the initial state here.
    f32x4 S[KT];
    int q0, q1;
    seg_range(p.st, n, a.nseg, 0, q0, q1);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        if (q1 > q0) {
            S[kt] = *reinterpret_cast<const f32x4*>(a.sloc + rec0 * (K * V) + (vt * KT + kt) * TILE + 4 * l);
        } else {
            S[kt] = zero4();
            if (p.h0) {
#pragma unroll
                for (int i = 0; i < 4; ++i) S[kt][i] = p.h0[soff + (int64_t)(16 * kt + 4 * g + i) * V];
            }
        }
    }
    // the chain, FIXUP_STAGE non-empty segments at a time
    int s = 1;
    while (s < target) {
        int step[FIXUP_STAGE], ns = 0;
#pragma unroll
        for (int b = 0; b < FIXUP_STAGE; ++b) {
            step[b] = 0;
            while (s < target) {
                seg_range(p.st, n, a.nseg, s, q0, q1);
                if (q1 > q0) break;
                ++s;
            }
            if (s < target) { step[b] = s++; ns = b + 1; }
        }
        f32x4 mq[FIXUP_STAGE][NQ], add[FIXUP_STAGE][KT];
#pragma unroll
        for (int b = 0; b < FIXUP_STAGE; ++b) {
            if (b < ns) {
                const float* mrec = a.mseg + (rec0 + step[b]) * (K * K) + wv * NQ * TILE + 4 * l;
                const float* srec = a.sloc + (rec0 + step[b]) * (K * V) + vt * KT * TILE + 4 * l;
#pragma unroll
                for (int i = 0; i < NQ; ++i) mq[b][i] = *reinterpret_cast<const f32x4*>(mrec + i * TILE);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) add[b][kt] = *reinterpret_cast<const f32x4*>(srec + kt * TILE);
            }
        }
        __syncthreads();                                  // the previous round's records have been used
#pragma unroll
        for (int b = 0; b < FIXUP_STAGE; ++b) {
            if (b < ns) {
#pragma unroll
                for (int i = 0; i < NQ; ++i) {
                    Split<T> q;
                    split(mq[b][i], q);
                    st_tile(sM[b][0] + (wv * NQ + i) * TILE, q.hi);
                    st_tile(sM[b][1] + (wv * NQ + i) * TILE, q.lo);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < FIXUP_STAGE; ++b) {
            if (b < ns) {
                // X^T <- X^T Q^T + A^T in split 2-byte products (three per tile pair: the error of fp32 products); tile
                // (out, in) of the record is at index out * KT + in
                Split<T> xs[KT];
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) split(S[kt], xs[kt]);
#pragma unroll
                for (int ko = 0; ko < KT; ++ko) {
                    f32x4 acc = add[b][ko];
#pragma unroll
                    for (int ki = 0; ki < KT; ++ki) {
                        Split<T> q;
                        q.hi = ld_tile(sM[b][0] + (ko * KT + ki) * TILE);
                        q.lo = ld_tile(sM[b][1] + (ko * KT + ki) * TILE);
                        acc = mm3(xs[ki], q, acc);
                    }
                    S[ko] = acc;
                }
            }
        }
    }
    if (target == a.nseg) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) p.ht[soff + (int64_t)(16 * kt + 4 * g + i) * V] = S[kt][i];
        return;
    }
    if (a.sin_out && part == 0) {
        float* so = a.sin_out + (rec0 + target) * (K * V) + vt * KT * TILE;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) *reinterpret_cast<f32x4*>(so + kt * TILE + 4 * l) = S[kt];
    }
    if (!a.gw) return;                                    // chaining only (the backward pass re-deriving the states)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) st_tile(sS + (vt * KT + kt) * TILE, to_frag<T>(S[kt]));
    __syncthreads();
    Frag<T> Sb[VT][KT];
#pragma unroll
    for (int j = 0; j < VT; ++j)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) Sb[j][kt] = ld_tile(sS + (j * KT + kt) * TILE);
    char* const st = stage[wv];
    for (int first = s0 + wv; first < s1; first += 4 * NB) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int cid = first + 4 * b;
            if (cid < s1) {
                const int64_t tok0 = bos + (int64_t)(cid - c0) * CH;
                const int len = (int)min((int64_t)CH, eos - tok0);
#pragma unroll
                for (int j = 0; j < VT; ++j) {
                    f32x4 o = OLr[b][j];
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) o = mm(G[b][kt], Sb[j][kt], o);
                    st_frag(reinterpret_cast<T*>(st + c * OROW) + 16 * j + 4 * g, to_frag<T>(o));
                }
                // whole rows, 16 bytes a lane (the wave's own staging area: LDS accesses of one wave complete in order)
                constexpr int LPR = V * (int)sizeof(T) / 16, RPI = 64 / LPR;
#pragma unroll
                for (int r0 = 0; r0 < CH; r0 += RPI) {
                    const int r = r0 + l / LPR, e = (l % LPR) * 16;
                    const i32x4 x = *reinterpret_cast<const i32x4*>(st + r * OROW + e);
                    if (r < len) *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(p.o + ((tok0 + r) * H + h) * V) + e) = x;
                }
            }
        }
        if (first + 4 * NB < s1) request(first + 4 * NB);
    }
}

}  // namespace hdla
