// chunk_grad kernel: everything of the backward pass that is local to one 16-token chunk.
//
// One wavefront per (chunk, head) fuses what the reference runs as five launches: the dA part of
// HRDPLR/bwd_triton.py:30-105, the dv kernel :239-290, the dqg/dkg/dbg/dw/dgk_last kernel :309-487, the WY
// backward :503-612, the score backward :627-883 and the log-decay gradient :899-948.  Its inputs are the
// original tensors, do, and per chunk the state entering it (h), the gradient of the state leaving it (dh),
// v_new and its gradient, all left in the workspace by the two scans.  Nothing but the seven gradients is
// written back.
//
// Two differences from the reference's algebra, both exact:
//  * the WY backward never forms d(Tm): with X = [w | u] = Tm R, R = [ag | A_ak v] one has dR = Tm^T dX and
//    dA_ab = mask(dR X^T), which replaces the Tm^T dTm Tm^T chain of bwd_triton.py:577-612;
//  * the score backward covers the whole 16 x 16 (x2 ranks) tile with MFMA products against the same
//    factorised operands as the forward pass instead of a serial per-column loop.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

constexpr int LDG = 36;

template <typename T, bool GKF32, int K, int V>
__global__ __launch_bounds__(64) void chunk_grad_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16, VT = V / 16;
    constexpr int SFS = blk_fwd(K, sizeof(T), false).SIZE / (int)sizeof(T);   // elements between slots of the scan block
    __shared__ __attribute__((aligned(16))) float sT[32 * LDG];   // 4608 bytes: stash of the transposed score-gradient tiles
    // do, v, v_new (2 ranks) and dv_new (2 ranks) of the chunk, [matrix][token][value], staged once: every one of
    // them is an operand of several products in every pass, and the working set of the resident waves is far
    // larger than the L2, so repeated global loads would mostly be repeated HBM reads
    constexpr int VP = V + 16 / (int)sizeof(T);                    // padded row, keeps 16-byte alignment
    __shared__ __attribute__((aligned(16))) T sTok[6 * CH * VP];
    // Results of 2-byte elements leave through LDS: a lane holds 8 bytes of a row, and 8-byte stores of four lanes
    // would write 32-byte pieces of rows, half of what HBM writes at once.  Two adjacent 16-column tiles are put
    // side by side in LDS and stored 16 bytes a lane, 64 contiguous bytes a row.
    constexpr bool STAGE_OUT = sizeof(T) == 2;
    constexpr int OPITCH = 80;                                     // bytes; 64 of data, padded against bank conflicts
    __shared__ __attribute__((aligned(16))) char sOut[STAGE_OUT ? 7 * CH * OPITCH : 16];

    const int cid = blockIdx.x, h = blockIdx.y;
    ChunkPos cp;
    if (!locate_chunk(p.st, cid, cp)) return;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    const bool rowok = c < cp.len;
    // Element offsets of the chunk's first row (uniform) and byte offsets of this lane's four elements in row
    // min(c, len-1) (rows past the end alias the last valid row and are masked by rowok); a/b rows are rank-minor.
    constexpr uint32_t ES = sizeof(T), GS = GKF32 ? 4 : 2;
    const int row = min(c, cp.len - 1);
    const int64_t qb = (cp.tok0 * H + h) * K, ab = (cp.tok0 * RANK * H + h) * K, vb = (cp.tok0 * H + h) * V;
    const uint32_t qe = (uint32_t)(row * H * K + 4 * g), ae = (uint32_t)(row * RANK * H * K + 4 * g);
    const uint32_t qo = qe * ES, go = qe * GS, ao0 = ae * ES, ao1 = ao0 + (uint32_t)(H * K) * ES;
    const uint32_t vo = (uint32_t)(row * H * V + 4 * g) * ES;
    const char* gkp = reinterpret_cast<const char*>(p.gk) + qb * GS;
    char* dgkp = reinterpret_cast<char*>(p.dgk) + qb * GS;
    const int64_t chw = (int64_t)h * p.st.nch + cid;
    const float scale = p.scale;
    const T* HC = p.ws.HC + chw * (K * V);
    const T* DHC = p.ws.DHC + chw * (K * V);
    const T* DVN = p.ws.DVN + chw * (2 * CH * V);
    const int blk = blockIdx.y * gridDim.x + blockIdx.x;
    PHASE_CLOCK(p, blk, 0);

    // q, k, a and gk of the chunk stay in registers for their second use in the last pass (a second load would
    // mostly be a second HBM read); bf16 operands only, fp32 ones would not fit next to the accumulators.  Their
    // loads are the first thing issued, so that they travel together with the staging loads below: a wave spends
    // most of its time waiting for memory, and every dependent round trip to HBM costs thousands of cycles.
    constexpr bool KEEP = sizeof(T) == 2;
    // The smallest shape also keeps the whole checkpoint of S (all its tile pairs) in registers from here to the
    // end: it is used three times (v_new, first and second pass over channel tiles) and a later read would mostly
    // come from HBM again; the other shapes read it tile by tile where it is used.
    constexpr bool PF = sizeof(T) == 2 && K == 64 && V == 64;
    constexpr int KT2 = KT / 2;
    Frag<T> hcall[PF ? KT2 : 1][PF ? VT : 1][2];
    if (PF) {
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp)
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) ld_pair(HC + (kp * VT + vt) * PAIR, hcall[PF ? kp : 0][PF ? vt : 0][0], hcall[PF ? kp : 0][PF ? vt : 0][1]);
    }
    Frag<T> rq[KEEP ? KT : 1], rk[KEEP ? KT : 1], ra[2][KEEP ? KT : 1];
    f32x4 rg[KEEP ? KT : 1];
    if (KEEP) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            rg[KEEP ? kt : 0] = ld_gk4<GKF32>(gkp + go + 16 * kt * GS, 0, rowok);
            rq[KEEP ? kt : 0] = ld_frag_sel(at(p.q + qb, qo + 16 * kt * ES), rowok);
            rk[KEEP ? kt : 0] = ld_frag_sel(at(p.k + qb, qo + 16 * kt * ES), rowok);
            ra[0][KEEP ? kt : 0] = ld_frag_sel(at(p.a + ab, ao0 + 16 * kt * ES), rowok);
            ra[1][KEEP ? kt : 0] = ld_frag_sel(at(p.a + ab, ao1 + 16 * kt * ES), rowok);
        }
    }
    const Frag<T> ident = ident_frag<T>();
    {
        // do and v: rows of the original tensors, 16 bytes per lane
        constexpr int EPL = 16 / (int)sizeof(T), LPR = V / EPL, RPI = 64 / LPR;    // elements/lane, lanes/row, rows/instr
        const int rr = l / LPR, e = (l % LPR) * EPL;
        typedef int i32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int r0 = 0; r0 < CH; r0 += RPI) {
                const int r = r0 + rr;
                const T* src = at((m == 0 ? p.dout : p.v) + vb, (uint32_t)(min(r, cp.len - 1) * H * V + e) * ES);
                i32x4 x = *reinterpret_cast<const i32x4*>(src);
                if (r >= cp.len) x = (i32x4){0, 0, 0, 0};
                *reinterpret_cast<i32x4*>(&sTok[(m * CH + r) * VP + e]) = x;
            }
        // dv_new: the reverse scan left it as fragments of the transposed tiles (rows value, inner token), the two
        // ranks of a value tile paired; one transposing product each gives the rows.
        // v_new is not checkpointed by the scan: v_new_s = w_s S + u_s is rebuilt here from the checkpoint of S, which
        // is stored as exactly the operand this product needs (fragments of S^T), with the same bf16 operands and
        // fp32 accumulation as in the scan.
        Frag<T> wf[2][KT];
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp)
                ld_pair(p.ws.W + chw * SFS + (s * (KT / 2) + kp) * PAIR, wf[s][2 * kp], wf[s][2 * kp + 1]);
#pragma unroll(sizeof(T) * V >= 512 ? 1 : VT)
        for (int vt = 0; vt < VT; ++vt) {
            Frag<T> u0, u1, y0, y1;
            ld_pair(p.ws.UT + (chw * VT + vt) * PAIR, u0, u1);
            ld_pair(DVN + vt * PAIR, y0, y1);
            f32x4 vn0 = zero4(), vn1 = zero4();
#pragma unroll
            for (int kp = 0; kp < KT / 2; ++kp) {
                Frag<T> h0, h1;
                if (PF) { h0 = hcall[PF ? kp : 0][PF ? vt : 0][0]; h1 = hcall[PF ? kp : 0][PF ? vt : 0][1]; }
                else ld_pair(HC + (kp * VT + vt) * PAIR, h0, h1);
                vn0 = mm(wf[0][2 * kp], h0, vn0);
                vn1 = mm(wf[1][2 * kp], h0, vn1);
                vn0 = mm(wf[0][2 * kp + 1], h1, vn0);
                vn1 = mm(wf[1][2 * kp + 1], h1, vn1);
            }
            vn0 += to_f32(transpose(u0, ident));
            vn1 += to_f32(transpose(u1, ident));
            T* dst = &sTok[c * VP + 16 * vt + 4 * g];
            st_frag(dst + 2 * CH * VP, to_frag<T>(vn0));
            st_frag(dst + 3 * CH * VP, to_frag<T>(vn1));
            st_frag(dst + 4 * CH * VP, transpose(y0, ident));
            st_frag(dst + 5 * CH * VP, transpose(y1, ident));
        }
    }
    auto tokf = [&](int m, int vt) __attribute__((always_inline)) { return ld_frag(&sTok[(m * CH + c) * VP + 16 * vt + 4 * g]); };
    // tmT[s][r] = F((Tm^{s r})^T): lane (g,c) reg i = Tm^{s r}[4g+i][c], stored in this form by the prep kernel
    Frag<T> tmT[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) ld_pair(p.ws.TM + chw * 1024 + s * PAIR, tmT[s][0], tmT[s][1]);
    __syncthreads();

    // ---- cumulative decays; A_qk^T and A_ak^T (rows j, inner i) -----------------------------------------------
    // (the decays are recomputed per channel tile wherever they are needed: a load and four DPP additions cost
    // less than keeping 2*K/16 vector registers alive across the kernel)
    f32x4 aqkT = zero4(), aakT[2] = {zero4(), zero4()};
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        const f32x4 g4 = KEEP ? rg[KEEP ? kt : 0] : ld_gk4<GKF32>(gkp + go + 16 * kt * GS, 0, rowok);
        const f32x4 gi = scan16_incl(g4), ge = gi - g4;
        const f32x4 m = bcast16(gi, MID);
        const f32x4 eq = exp4<T>(gi - m), ek = exp4<T>(m - gi), ea = exp4<T>(ge - m);
        const Frag<T> fq = KEEP ? rq[KEEP ? kt : 0] : ld_frag_sel(at(p.q + qb, qo + 16 * kt * ES), rowok);
        const Frag<T> fk = KEEP ? rk[KEEP ? kt : 0] : ld_frag_sel(at(p.k + qb, qo + 16 * kt * ES), rowok);
        const Frag<T> fa0 = KEEP ? ra[0][KEEP ? kt : 0] : ld_frag_sel(at(p.a + ab, ao0 + 16 * kt * ES), rowok);
        const Frag<T> fa1 = KEEP ? ra[1][KEEP ? kt : 0] : ld_frag_sel(at(p.a + ab, ao1 + 16 * kt * ES), rowok);
        const f32x4 q4 = to_f32(fq), k4 = to_f32(fk), a0 = to_f32(fa0), a1 = to_f32(fa1);
        const Frag<T> qh = to_frag<T>(q4 * eq * scale), kh = to_frag<T>(k4 * ek);
        aqkT = mm(kh, qh, aqkT);
        aakT[0] = mm(kh, to_frag<T>(a0 * ea), aakT[0]);
        aakT[1] = mm(kh, to_frag<T>(a1 * ea), aakT[1]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {          // row j = c, inner i = 4g+i
        const int ii = 4 * g + i;
        if (!(c <= ii)) aqkT[i] = 0.f;
        if (!(c < ii)) { aakT[0][i] = 0.f; aakT[1][i] = 0.f; }
    }
    const Frag<T> aqkTf = to_frag<T>(aqkT);
    const Frag<T> aakTf[2] = {to_frag<T>(aakT[0]), to_frag<T>(aakT[1])};

    // In the second pass the checkpoint of the state gradient arrives a pair of channel tiles ahead of its use:
    // [buffer][value tile][tile of the pair].
    Frag<T> dhp[PF ? 2 : 1][PF ? VT : 1][2];
    auto fetch_pairs = [&](const T* src, Frag<T> (&dst)[PF ? VT : 1][2], int kp) __attribute__((always_inline)) {
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) ld_pair(src + (kp * VT + vt) * PAIR, dst[PF ? vt : 0][0], dst[PF ? vt : 0][1]);
    };
    PHASE_CLOCK(p, blk, 1);
    // ---- products over the value dimension -------------------------------------------------------------------
    f32x4 dAqk = zero4(), dAqb[2] = {zero4(), zero4()}, dAak[2] = {zero4(), zero4()};
    f32x4 dAab[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
    f32x4 dv[VT];
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
        const Frag<T> doN = tokf(0, vt);
        const Frag<T> vN = tokf(1, vt);
        const Frag<T> vnN[2] = {tokf(2, vt), tokf(3, vt)};
        dAqk = mm(doN, vN, dAqk);
        dAqb[0] = mm(doN, vnN[0], dAqb[0]);
        dAqb[1] = mm(doN, vnN[1], dAqb[1]);
        const Frag<T> doT = transpose(doN, ident);
        Frag<T> dvnT[2];                                  // as the reverse scan left them: rows value, inner token
        ld_pair(DVN + vt * PAIR, dvnT[0], dvnT[1]);
        Frag<T> dMf[2], dMTf[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            f32x4 x = mm(tmT[0][r], dvnT[0], zero4());
            x = mm(tmT[1][r], dvnT[1], x);
            dMf[r] = to_frag<T>(x);                       // dM_r   rows i, inner value
            f32x4 y = mm(dvnT[0], tmT[0][r], zero4());
            y = mm(dvnT[1], tmT[1][r], y);
            dMTf[r] = to_frag<T>(y);                      // dM_r^T rows value, inner i
        }
        const Frag<T> uN[2] = {transpose(ld_pair_one(p.ws.UT + (chw * VT + vt) * PAIR, 0), ident),
                               transpose(ld_pair_one(p.ws.UT + (chw * VT + vt) * PAIR, 1), ident)};
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            dAak[r] = mm(dMf[r], vN, dAak[r]);
            dAab[r][0] = mm(dMf[r], uN[0], dAab[r][0]);
            dAab[r][1] = mm(dMf[r], uN[1], dAab[r][1]);
        }
        f32x4 x = mm(aqkTf, doT, zero4());
        x = mm(aakTf[0], dMTf[0], x);
        x = mm(aakTf[1], dMTf[1], x);
        dv[vt] = x;                                       // rows token, inner value; kg dS is added below
    }

    PHASE_CLOCK(p, blk, 2);
    // ---- first pass over channel tiles: dw -> dag -> the w part of dA_ab (dag itself is rebuilt in pass two) ----
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        f32x4 dwT[2] = {zero4(), zero4()};                // rows channel, inner token
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const Frag<T> Sf = transpose(PF ? hcall[PF ? kt / 2 : 0][PF ? vt : 0][kt & 1]
                                            : ld_pair_one(HC + ((kt / 2) * VT + vt) * PAIR, kt & 1), ident);
            dwT[0] = mm(Sf, tokf(4, vt), dwT[0]);
            dwT[1] = mm(Sf, tokf(5, vt), dwT[1]);
        }
        const Frag<T> dwTf[2] = {to_frag<T>(dwT[0]), to_frag<T>(dwT[1])};
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            f32x4 x = mm(tmT[0][r], dwTf[0], zero4());
            x = mm(tmT[1][r], dwTf[1], x);                // dag_r: rows token, inner channel
            const Frag<T> dagf = to_frag<T>(x);
            dAab[r][0] = mm(dagf, ld_pair_one(p.ws.W + chw * SFS + (0 * (KT / 2) + kt / 2) * PAIR, kt & 1), dAab[r][0]);
            dAab[r][1] = mm(dagf, ld_pair_one(p.ws.W + chw * SFS + (1 * (KT / 2) + kt / 2) * PAIR, kt & 1), dAab[r][1]);
        }
    }

    // for the second pass: the first pair of S and dS tiles, and all of b (used there only), requested now
    Frag<T> rb[2][KEEP ? KT : 1];
    if (PF) fetch_pairs(DHC, dhp[0], 0);
    if (KEEP) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            rb[0][KEEP ? kt : 0] = ld_frag_sel(at(p.b + ab, ao0 + 16 * kt * ES), rowok);
            rb[1][KEEP ? kt : 0] = ld_frag_sel(at(p.b + ab, ao1 + 16 * kt * ES), rowok);
        }
    }
    PHASE_CLOCK(p, blk, 3);
    // ---- masks; both orientations of the nine score-gradient tiles --------------------------------------------
#pragma unroll
    for (int i = 0; i < 4; ++i) {          // row i = c, inner j = 4g+i
        const int j = 4 * g + i;
        if (!(j <= c)) { dAqk[i] = 0.f; dAqb[0][i] = 0.f; dAqb[1][i] = 0.f; }
        if (!(j < c)) { dAak[0][i] = 0.f; dAak[1][i] = 0.f; dAab[0][0][i] = 0.f; dAab[0][1][i] = 0.f; dAab[1][0][i] = 0.f; dAab[1][1][i] = 0.f; }
    }
    // The transposed tiles are needed once per channel tile of the second pass.  For 2-byte elements the nine of
    // them are kept in LDS (4608 bytes) and read back where used: 18 registers less across the second pass.
    constexpr bool STASH = sizeof(T) == 2;
    T* stash = reinterpret_cast<T*>(sT);
    const Frag<T> fAqk = to_frag<T>(dAqk);
    Frag<T> fAqb[2], fAak[2], fAab[2][2];
    Frag<T> rT[STASH ? 1 : 9];                             // transposes kept in registers otherwise
    auto putT = [&](int idx, Frag<T> f) __attribute__((always_inline)) {
        const Frag<T> t = transpose(f, ident);
        if (STASH) st_tile(stash + idx * TILE, t);
        else rT[STASH ? 0 : idx] = t;
    };
    auto getT = [&](int idx) __attribute__((always_inline)) { return STASH ? ld_tile(stash + idx * TILE) : rT[STASH ? 0 : idx]; };
    // indices: 0 A_qk, 1+s A_qb^s, 3+s A_ak^s, 5+2r+s A_ab^{r s}
    putT(0, fAqk);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        fAqb[s] = to_frag<T>(dAqb[s]); putT(1 + s, fAqb[s]);
        fAak[s] = to_frag<T>(dAak[s]); putT(3 + s, fAak[s]);
#pragma unroll
        for (int r = 0; r < 2; ++r) { fAab[r][s] = to_frag<T>(dAab[r][s]); putT(5 + 2 * r + s, fAab[r][s]); }
    }

    // put(m, half, f): tile f of output m into column half `half`; flush(m, base, byte0): the 16 x 32 block out
    auto put = [&](int m, int half, Frag<T> f) __attribute__((always_inline)) {
        st_frag(reinterpret_cast<T*>(sOut + (m * CH + c) * OPITCH + half * 32) + 4 * g, f);
    };
    auto flush = [&](int m, T* ubase, uint32_t row_pitch_bytes, uint32_t byte0) __attribute__((always_inline)) {
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        const int r = l >> 2, piece = l & 3;
        const i32x4 x = *reinterpret_cast<const i32x4*>(sOut + (m * CH + r) * OPITCH + piece * 16);
        if (r < cp.len) *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(ubase) + (uint32_t)r * row_pitch_bytes + byte0 + piece * 16) = x;
    };
    PHASE_CLOCK(p, blk, 4);
    // ---- second pass over channel tiles: state products, score backward, final gradients ----------------------
#pragma unroll(KEEP ? KT : 1)
    for (int kt = 0; kt < KT; ++kt) {
        if (PF && !(kt & 1) && kt / 2 + 1 < KT2) fetch_pairs(DHC, dhp[PF ? (kt / 2 + 1) & 1 : 0], kt / 2 + 1);
        // (a) what the loop over value tiles needs: only kg of this channel tile
        const f32x4 g4 = KEEP ? rg[KEEP ? kt : 0] : ld_gk4<GKF32>(gkp + go + 16 * kt * GS, 0, rowok);
        const f32x4 gi = scan16_incl(g4);
        const f32x4 gl = bcast16(gi, CH - 1);
        const f32x4 edn = exp4<T>(gl - gi);
        const f32x4 k4 = to_f32(KEEP ? rk[KEEP ? kt : 0] : ld_frag_sel(at(p.k + qb, qo + 16 * kt * ES), rowok));
        const f32x4 kg4 = k4 * edn;
        const Frag<T> kgf = to_frag<T>(kg4);

        f32x4 dqg = zero4(), dkg = zero4(), dbg[2] = {zero4(), zero4()};
        f32x4 dwT[2] = {zero4(), zero4()};                 // dw_s^T for this channel tile (rows channel, inner token)
        float hh = 0.f;                                    // partial of sum_v S * dS for channel 16kt + c
#pragma unroll(sizeof(T) == 2 ? VT : 2)
        for (int vt = 0; vt < VT; ++vt) {
            // the scans checkpoint S and dS as fragments of the transposed tiles (rows value, inner channel)
            const Frag<T> dST = PF ? dhp[PF ? (kt / 2) & 1 : 0][PF ? vt : 0][kt & 1] : ld_pair_one(DHC + ((kt / 2) * VT + vt) * PAIR, kt & 1);
            const Frag<T> Sf = transpose(PF ? hcall[PF ? kt / 2 : 0][PF ? vt : 0][kt & 1]
                                            : ld_pair_one(HC + ((kt / 2) * VT + vt) * PAIR, kt & 1), ident);
            const Frag<T> dSf = transpose(dST, ident);
            const Frag<T> doN = tokf(0, vt);
            const Frag<T> vN = tokf(1, vt);
            dqg = mm(doN, Sf, dqg);
            dwT[0] = mm(Sf, tokf(4, vt), dwT[0]);
            dwT[1] = mm(Sf, tokf(5, vt), dwT[1]);
            dkg = mm(vN, dSf, dkg);
            dbg[0] = mm(tokf(2, vt), dSf, dbg[0]);
            dbg[1] = mm(tokf(3, vt), dSf, dbg[1]);
            const f32x4 s4 = to_f32(Sf), d4 = to_f32(dSf);
            hh += s4[0] * d4[0] + s4[1] * d4[1] + s4[2] * d4[2] + s4[3] * d4[3];
            dv[vt] = mm(kgf, dST, dv[vt]);
        }
        hh += __shfl_xor(hh, 16);
        hh += __shfl_xor(hh, 32);
        f32x4 hh4;
#pragma unroll
        for (int i = 0; i < 4; ++i) hh4[i] = __shfl(hh, 4 * g + i);

        const Frag<T> dwTf[2] = {to_frag<T>(dwT[0]), to_frag<T>(dwT[1])};
        f32x4 dag[2];                                      // dag_r = sum_s (Tm^{s r})^T dw_s, rows token, inner channel
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            dag[r] = mm(tmT[0][r], dwTf[0], zero4());
            dag[r] = mm(tmT[1][r], dwTf[1], dag[r]);
        }
        // (b) the factorised operands and decay factors of this channel tile, for the score backward
        const f32x4 ge = gi - g4;
        const f32x4 m = bcast16(gi, MID);
        const f32x4 eq = exp4<T>(gi - m), ek = exp4<T>(m - gi), ea = exp4<T>(ge - m);
        const f32x4 egi = exp4<T>(gi), ege = exp4<T>(ge);
        const f32x4 q4 = to_f32(KEEP ? rq[KEEP ? kt : 0] : ld_frag_sel(at(p.q + qb, qo + 16 * kt * ES), rowok));
        const f32x4 a4[2] = {to_f32(KEEP ? ra[0][KEEP ? kt : 0] : ld_frag_sel(at(p.a + ab, ao0 + 16 * kt * ES), rowok)),
                             to_f32(KEEP ? ra[1][KEEP ? kt : 0] : ld_frag_sel(at(p.a + ab, ao1 + 16 * kt * ES), rowok))};
        const f32x4 b4[2] = {to_f32(KEEP ? rb[0][KEEP ? kt : 0] : ld_frag_sel(at(p.b + ab, ao0 + 16 * kt * ES), rowok)),
                             to_f32(KEEP ? rb[1][KEEP ? kt : 0] : ld_frag_sel(at(p.b + ab, ao1 + 16 * kt * ES), rowok))};
        const Frag<T> qhT = transpose(to_frag<T>(q4 * eq * scale), ident), khT = transpose(to_frag<T>(k4 * ek), ident);
        const Frag<T> ahT[2] = {transpose(to_frag<T>(a4[0] * ea), ident), transpose(to_frag<T>(a4[1] * ea), ident)};
        const Frag<T> bhT[2] = {transpose(to_frag<T>(b4[0] * ek), ident), transpose(to_frag<T>(b4[1] * ek), ident)};
        const f32x4 bg4[2] = {b4[0] * edn, b4[1] * edn};
        f32x4 dqh = mm(fAqk, khT, zero4());
        dqh = mm(fAqb[0], bhT[0], dqh);
        dqh = mm(fAqb[1], bhT[1], dqh);
        f32x4 dkh = mm(getT(0), qhT, zero4());
        dkh = mm(getT(3), ahT[0], dkh);
        dkh = mm(getT(4), ahT[1], dkh);
        f32x4 dah[2], dbh[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            f32x4 x = mm(fAak[r], khT, zero4());
            x = mm(fAab[r][0], bhT[0], x);
            x = mm(fAab[r][1], bhT[1], x);
            dah[r] = x;
            f32x4 y = mm(getT(1 + r), qhT, zero4());          // here r plays the role of the b rank s
            y = mm(getT(5 + r), ahT[0], y);
            y = mm(getT(7 + r), ahT[1], y);
            dbh[r] = y;
        }
        const f32x4 dq = (dqh * eq + dqg * egi) * scale;
        const f32x4 dk = dkh * ek + dkg * edn;
        const f32x4 da[2] = {dah[0] * ea + dag[0] * ege, dah[1] * ea + dag[1] * ege};
        const f32x4 db[2] = {dbh[0] * ek + dbg[0] * edn, dbh[1] * ek + dbg[1] * edn};
        const f32x4 Dge = da[0] * a4[0] + da[1] * a4[1];
        const f32x4 Dgi = dq * q4 - dk * k4 - db[0] * b4[0] - db[1] * b4[1];
        const f32x4 dgl = exp4<T>(gl) * hh4 + sum16(dkg * kg4 + dbg[0] * bg4[0] + dbg[1] * bg4[1]);
        const f32x4 dg = rscan16_incl(Dgi + Dge) - Dge + dgl;
        if (STAGE_OUT) {
            const int half = kt & 1;
            put(0, half, to_frag<T>(dq));
            put(1, half, to_frag<T>(dk));
            put(2, half, to_frag<T>(da[0]));
            put(3, half, to_frag<T>(da[1]));
            put(4, half, to_frag<T>(db[0]));
            put(5, half, to_frag<T>(db[1]));
            if (!GKF32) put(6, half, to_frag<T>(dg));
            else if (rowok) st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
            if (half) {
                const uint32_t qpitch = (uint32_t)(H * K) * ES, apitch = qpitch * RANK, b0 = (uint32_t)(16 * (kt - 1)) * ES;
                flush(0, p.dq + qb, qpitch, b0);
                flush(1, p.dk + qb, qpitch, b0);
                flush(2, p.da + ab, apitch, b0);
                flush(3, p.da + ab, apitch, b0 + qpitch);
                flush(4, p.db + ab, apitch, b0);
                flush(5, p.db + ab, apitch, b0 + qpitch);
                if (!GKF32) flush(6, reinterpret_cast<T*>(dgkp), qpitch, b0);
            }
        } else if (rowok) {
            st_frag(at(p.dq + qb, qo + 16 * kt * ES), to_frag<T>(dq));
            st_frag(at(p.dk + qb, qo + 16 * kt * ES), to_frag<T>(dk));
            st_frag(at(p.da + ab, ao0 + 16 * kt * ES), to_frag<T>(da[0]));
            st_frag(at(p.da + ab, ao1 + 16 * kt * ES), to_frag<T>(da[1]));
            st_frag(at(p.db + ab, ao0 + 16 * kt * ES), to_frag<T>(db[0]));
            st_frag(at(p.db + ab, ao1 + 16 * kt * ES), to_frag<T>(db[1]));
            st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
        }
    }
    if (STAGE_OUT) {
#pragma unroll
        for (int vt = 0; vt < VT; vt += 2) {
            put(0, 0, to_frag<T>(dv[vt]));
            put(0, 1, to_frag<T>(dv[vt + 1]));
            flush(0, p.dv + vb, (uint32_t)(H * V) * ES, (uint32_t)(16 * vt) * ES);
        }
    } else if (rowok) {
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) st_frag(at(p.dv + vb, vo + 16 * vt * ES), to_frag<T>(dv[vt]));
    }
    PHASE_CLOCK(p, blk, 5);
}

template <typename T, int K, int V>
static hipError_t launch_chunk_grad_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.st.nch, a.H), block(64);
    constexpr bool kAlwaysF32 = sizeof(T) == 4;
    if (kAlwaysF32 || a.gk_f32) hipLaunchKernelGGL((chunk_grad_kernel<T, true, K, V>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((chunk_grad_kernel<T, kAlwaysF32, K, V>), grid, block, 0, stream, a);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_chunk_grad(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_chunk_grad_kv<T, 64, 64>(a, stream);
    if (K == 128 && V == 128) return launch_chunk_grad_kv<T, 128, 128>(a, stream);
    if (K == 64 && V == 128) return launch_chunk_grad_kv<T, 64, 128>(a, stream);
    if (K == 128 && V == 64) return launch_chunk_grad_kv<T, 128, 64>(a, stream);
    return hipErrorInvalidValue;
}
template hipError_t launch_chunk_grad<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_chunk_grad<float>(const ChunkArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
