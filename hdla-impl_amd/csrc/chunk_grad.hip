// chunk_grad kernel: everything of the backward pass that is local to one 16-token chunk.
//
// One workgroup of four wavefronts per (chunk, head) fuses what the reference runs as five launches: the dA part of
// HRDPLR/bwd_triton.py:30-105, the dv kernel :239-290, the dqg/dkg/dbg/dw/dgk_last kernel :309-487, the WY
// backward :503-612, the score backward :627-883 and the log-decay gradient :899-948.  Its inputs are the
// original tensors, do, and per chunk the state entering it (h), the gradient of the state leaving it (dh) and
// the gradient of v_new, left in the workspace by the two scans.  Nothing but the seven gradients is written back.
//
// Two differences from the reference's algebra, both exact:
//  * the WY backward never forms d(Tm): with X = [w | u] = Tm R, R = [ag | A_ak v] one has dR = Tm^T dX and
//    dA_ab = mask(dR X^T), which replaces the Tm^T dTm Tm^T chain of bwd_triton.py:577-612;
//  * the score backward covers the whole 16 x 16 (x2 ranks) tile with MFMA products against the same
//    factorised operands as the forward pass instead of a serial per-column loop.
//
// Division of the work: every product here contracts over channels or over value columns, so wave w owns the
// channel tiles kt = w*KT/4 .. and the value tiles vt = w*VT/4 ..; what is summed over the other dimension (the
// score tiles, their gradients, dv) is exchanged through LDS, with five workgroup barriers in all.  One wave per
// chunk would hold the whole chunk in registers, at one wave per SIMD, and nothing would overlap its arithmetic
// with the memory round trips of its neighbours; four waves on a quarter each leave room for two or three
// workgroups per compute unit.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

constexpr int NW = 4;     // wavefronts per (chunk, head)

typedef int i32x4 __attribute__((ext_vector_type(4)));

// LDS of a workgroup (byte offsets)
template <typename T, int K, int V> struct CgLds {
    static constexpr int ES = sizeof(T);
    // do, v, v_new (2 ranks), dv_new (2 ranks) of the chunk, [matrix][token][value], rows padded by 16 bytes
    static constexpr int VP = V + 16 / ES;
    static constexpr int TOK = 0, TOK_B = 6 * CH * VP * ES;
    // first, per wave: its part of A_qk^T, A_ak^T (2 ranks), fp32 tiles in fragment order (read between barriers 1
    // and 2); later the nine score-gradient tiles, as fragments and as fragments of their transposes (written
    // between barriers 2 and 3)
    static constexpr int SCORE = TOK + TOK_B, SCORE_B = NW * 3 * 1024, FIN = SCORE, FIN_B = 18 * TILE * ES;
    // kg of every channel tile (fragments), for dv
    static constexpr int KG = SCORE + (SCORE_B > FIN_B ? SCORE_B : FIN_B), KG_B = (K / 16) * TILE * ES;
    // first: the parts of the nine tiles (fp32), summed in two rounds through NW/2 slots; later, for 2-byte elements: the rows of the seven
    // gradients, so that they leave as whole rows (a lane holds 8 bytes of a row; 8-byte stores of four lanes
    // would write 32-byte pieces, half of what HBM writes at once)
    static constexpr bool STAGE_OUT = ES == 2;
    static constexpr int OPK = K * ES + 16, OPV = V * ES + 16;       // padded rows
    static constexpr int PART_B = (NW / 2) * 9 * 1024, OUT_B = STAGE_OUT ? (7 * OPK + OPV) * CH : 0;
    // per wave and token: three partial sums over channels of the backward of the HDLA parameterisation
    static constexpr int RED = KG + KG_B, RED_B = NW * 3 * CH * 4;
    static constexpr int R1 = RED + RED_B, R1_B = PART_B > OUT_B ? PART_B : OUT_B;
    static constexpr int BYTES = R1 + R1_B;
};

// waves per SIMD asked of the compiler (lowest, highest): three workgroups per compute unit for the smallest 2-byte
// shape, two for the other 2-byte shapes
template <typename T, bool GKF32, int K, int V, bool HD> constexpr int cg_waves(bool highest) {
    const bool small = sizeof(T) * K * V <= 2 * 64 * 64;
    if (sizeof(T) != 2) return highest ? 2 : 1;
    if (HD && GKF32 && small) return 2;                   // fp32 decay next to 2-byte inputs: four more registers a tile
    return small ? 3 : 2;
}

template <typename T, bool GKF32, int K, int V, bool HD>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(cg_waves<T, GKF32, K, V, HD>(false), cg_waves<T, GKF32, K, V, HD>(true)))) void chunk_grad_kernel(ChunkArgs<T> p) {
    constexpr int KT = K / 16, VT = V / 16, KT2 = KT / 2, KTW = KT / NW, VTW = VT / NW;
    static_assert(KT % NW == 0 && VT % NW == 0 && (KTW == 1 || KTW == 2), "a wave owns one channel tile or one stored pair");
    typedef CgLds<T, K, V> L;
    constexpr int VP = L::VP;
    constexpr bool STAGE_OUT = L::STAGE_OUT;
    constexpr int SFS = blk_fwd(K, sizeof(T), false).SIZE / (int)sizeof(T);   // elements between slots of the scan block
    __shared__ __attribute__((aligned(16))) char smem[L::BYTES];
    T* const sTok = reinterpret_cast<T*>(smem + L::TOK);
    float* const sScore = reinterpret_cast<float*>(smem + L::SCORE);
    T* const sKg = reinterpret_cast<T*>(smem + L::KG);
    T* const sFin = reinterpret_cast<T*>(smem + L::FIN);
    float* const sRed = reinterpret_cast<float*>(smem + L::RED);
    float* const sPart = reinterpret_cast<float*>(smem + L::R1);
    char* const sOut = smem + L::R1;

    // Which of the two indices runs fastest over the workgroups decides which rows of the [token][head][channel]
    // tensors the workgroups resident at one time touch.  Measured: with rows of 4 KiB and more, neighbouring
    // workgroups should be the heads of one chunk (together they read whole rows; chunk-fastest, all of them would
    // touch the same few hundred bytes of every row, a fraction of the HBM channels); with shorter rows the chunks
    // of one head, whose workspace records are contiguous.
    const bool head_fastest = (uint32_t)(p.H * K) * sizeof(T) >= 4096;
    const int cid = head_fastest ? blockIdx.x / p.H : blockIdx.x % p.st.nch;
    const int h = head_fastest ? blockIdx.x % p.H : blockIdx.x / p.st.nch;
    ChunkPos cp;
    if (!locate_chunk(p.st, cid, cp)) return;                 // uniform over the workgroup
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
    const T* Wb = p.ws.W + chw * SFS;
    const int kt0 = w * KTW, vt0 = w * VTW;                   // first own channel tile / value tile

    // ---- everything the wave reads from global memory is requested here, before any arithmetic -----------------
    // (the large shapes cannot hold all of it at once at two waves per SIMD: there the tiles of S and dS that are
    // used later are requested later, each a phase of arithmetic ahead of its first use)
    Frag<T> rq[KTW], rk[KTW], ra[2][KTW], rb[2][KTW];          // own channel tiles of the inputs
    f32x4 rg[KTW];
#pragma unroll
    for (int j = 0; j < KTW; ++j) {
        const uint32_t ko = 16 * (kt0 + j);
        rg[j] = ld_gk4<GKF32>(gkp + go + ko * GS, 0, rowok);
        rq[j] = ld_frag_sel(at(p.q + qb, qo + ko * ES), rowok);
        rk[j] = ld_frag_sel(at(p.k + qb, qo + ko * ES), rowok);
        if (!HD) {
            ra[0][j] = ld_frag_sel(at(p.a + ab, ao0 + ko * ES), rowok);
            ra[1][j] = ld_frag_sel(at(p.a + ab, ao1 + ko * ES), rowok);
        }
    }
    auto load_b = [&]() __attribute__((always_inline)) {       // b is used in the second pass only
        if (HD) return;
#pragma unroll
        for (int j = 0; j < KTW; ++j) {
            const uint32_t ko = 16 * (kt0 + j);
            rb[0][j] = ld_frag_sel(at(p.b + ab, ao0 + ko * ES), rowok);
            rb[1][j] = ld_frag_sel(at(p.b + ab, ao1 + ko * ES), rowok);
        }
    };
    // rows of do and v: 16 bytes a lane, the waves take turns
    constexpr int EPL = 16 / (int)sizeof(T), LPR = V / EPL, RPI = 64 / LPR, NRI = 2 * CH / RPI;   // elements/lane, lanes/row, rows/instr
    static_assert(NRI % NW == 0, "");
    i32x4 rows[NRI / NW];
#pragma unroll
    for (int j = 0; j < NRI / NW; ++j) {
        const int i = w + j * NW, m = i / (CH / RPI), r = (i % (CH / RPI)) * RPI + l / LPR;
        rows[j] = *reinterpret_cast<const i32x4*>(at((m == 0 ? p.dout : p.v) + vb, (uint32_t)(min(r, cp.len - 1) * H * V + (l % LPR) * EPL) * ES));
    }
    // the scans checkpoint S and dS as fragments of the transposed tiles (rows value, inner channel), tile pairs
    // [channel pair][value tile]: pair_of(X, kp, vt)
    auto own_kt_tiles = [&](const T* X, Frag<T> (&dst)[KTW][VT]) __attribute__((always_inline)) {
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            if (KTW == 2) ld_pair(X + (w * VT + vt) * PAIR, dst[0][vt], dst[KTW - 1][vt]);
            else dst[0][vt] = ld_pair_one(X + ((w >> 1) * VT + vt) * PAIR, w & 1);
        }
    };
    // one of the own channel tiles only (the large shapes request the second one when the first has been used)
    auto own_kt_tile = [&](const T* X, Frag<T> (&dst)[VT], int j) __attribute__((always_inline)) {
#pragma unroll
        for (int vt = 0; vt < VT; ++vt)
            dst[vt] = KTW == 2 ? ld_pair_one(X + (w * VT + vt) * PAIR, j) : ld_pair_one(X + ((w >> 1) * VT + vt) * PAIR, w & 1);
    };
    auto own_vt_tiles = [&](const T* X, Frag<T> (&dst)[VTW][KT]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < VTW; ++j)
#pragma unroll
            for (int kp = 0; kp < KT2; ++kp) ld_pair(X + (kp * VT + vt0 + j) * PAIR, dst[j][2 * kp], dst[j][2 * kp + 1]);
    };
    Frag<T> wf[2][KT], wk[2][KTW];                             // w: all of it (v_new), and the own channel tiles
    auto own_w_tiles = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (KTW == 2) ld_pair(Wb + (s * KT2 + w) * PAIR, wk[s][0], wk[s][KTW - 1]);
            else wk[s][0] = ld_pair_one(Wb + (s * KT2 + (w >> 1)) * PAIR, w & 1);
        }
    };
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int kp = 0; kp < KT2; ++kp) ld_pair(Wb + (s * KT2 + kp) * PAIR, wf[s][2 * kp], wf[s][2 * kp + 1]);
    Frag<T> hv[VTW][KT], hk[KTW][VT], dhv[VTW][KT], dhk[KTW][VT];
    constexpr bool EARLY = sizeof(T) * K * V <= 2 * 64 * 64;
    own_vt_tiles(HC, hv);
    if (EARLY) { own_kt_tiles(HC, hk); own_w_tiles(); }
    Frag<T> ut[VTW][2], yt[VTW][2];                            // u^T and dv_new^T of the own value tiles, both ranks
#pragma unroll
    for (int j = 0; j < VTW; ++j) {
        ld_pair(p.ws.UT + (chw * VT + vt0 + j) * PAIR, ut[j][0], ut[j][1]);
        ld_pair(DVN + (vt0 + j) * PAIR, yt[j][0], yt[j][1]);
    }
    // tmT[s][r] = F((Tm^{s r})^T): lane (g,c) reg i = Tm^{s r}[4g+i][c], stored in this form by the prep kernel
    Frag<T> tmT[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) ld_pair(p.ws.TM + chw * 1024 + s * PAIR, tmT[s][0], tmT[s][1]);
    if (EARLY) { own_kt_tiles(DHC, dhk); own_vt_tiles(DHC, dhv); load_b(); }

    // HDLA parameterisation (hdla_custom.py:19-43): a_1 = -beta k, a_2 = beta k (beta s - f), b_1 = f k, b_2 = k with
    // f = exp(gk) and s = sum over ALL channels of k^2 f.  A wave has a quarter of the channels: the waves exchange their
    // parts of s with the parts of the score tiles below, and until then nothing may depend on a_2.
    float beta_t = 0.f, s_t = 0.f;
    if (HD) beta_t = rowok ? ld_elem(p.beta + (cp.tok0 + row) * H + h) : 0.f;
    // a and b of the own channel tiles as the products take them: as loaded, or (HDLA parameterisation) formed on the
    // spot from k, gk, beta and s, which costs a few instructions and no registers in between
    auto a_of = [&](int r, int j) __attribute__((always_inline)) {
        if (!HD) return ra[r][j];
        const f32x4 kk = to_f32(rk[j]);
        return r == 0 ? to_frag<T>(kk * (-beta_t)) : to_frag<T>(kk * ((beta_t * s_t - exp4<T>(rg[j])) * beta_t));
    };
    auto b_of = [&](int r, int j) __attribute__((always_inline)) {
        if (!HD) return rb[r][j];
        return r == 0 ? to_frag<T>(exp4<T>(rg[j]) * to_f32(rk[j])) : rk[j];
    };
    const Frag<T> ident = ident_frag<T>();

    // ---- own channel tiles: part of A_qk^T and A_ak^T (rows j, inner i); kg for everybody ------------------------
    {
        // HDLA parameterisation: A_ak^r[i][j] = sum_c a_r[i][c] ea k^[j][c] with a_1 = -beta_i k, a_2 = beta_i^2 s_i k -
        // beta_i f k: the two tiles exchanged are X1 = (k ea) k^^T and X2 = (k f ea) k^^T, which need neither beta nor
        // s, and A_ak^1 = -beta X1, A_ak^2 = beta^2 s X1 - beta X2 follow from the sums (scaled along the inner index i)
        f32x4 aqkT = zero4(), aakT[2] = {zero4(), zero4()};
        float sp = 0.f;
#pragma unroll
        for (int j = 0; j < KTW; ++j) {
            const f32x4 g4 = rg[j];
            const f32x4 gi = scan16_incl(g4), ge = gi - g4;
            const f32x4 m = bcast16(gi, MID);
            const f32x4 eq = exp4<T>(gi - m), ek = exp4<T>(m - gi), ea = exp4<T>(ge - m);
            const f32x4 q4 = to_f32(rq[j]), k4 = to_f32(rk[j]);
            const Frag<T> qh = to_frag<T>(q4 * eq * scale), kh = to_frag<T>(k4 * ek);
            aqkT = mm(kh, qh, aqkT);
            if (HD) {
                const f32x4 f4 = exp4<T>(g4), kea = k4 * ea, kf = k4 * k4 * f4;
                aakT[0] = mm(kh, to_frag<T>(kea), aakT[0]);
                aakT[1] = mm(kh, to_frag<T>(kea * f4), aakT[1]);
                sp += kf[0] + kf[1] + kf[2] + kf[3];
            } else {
                aakT[0] = mm(kh, to_frag<T>(to_f32(ra[0][j]) * ea), aakT[0]);
                aakT[1] = mm(kh, to_frag<T>(to_f32(ra[1][j]) * ea), aakT[1]);
            }
            const f32x4 edn = exp4<T>(bcast16(gi, CH - 1) - gi);
            st_tile(sKg + (kt0 + j) * TILE, to_frag<T>(k4 * edn));
        }
        if (HD) {
            sp = sum_groups(sp);
            if (g == 0) { sRed[(w * 3 + 0) * CH + c] = sp; sRed[(w * 3 + 1) * CH + c] = beta_t; }
        }
        *reinterpret_cast<f32x4*>(sScore + ((w * 3 + 0) * 64 + l) * 4) = aqkT;
        *reinterpret_cast<f32x4*>(sScore + ((w * 3 + 1) * 64 + l) * 4) = aakT[0];
        *reinterpret_cast<f32x4*>(sScore + ((w * 3 + 2) * 64 + l) * 4) = aakT[1];
    }
    // ---- staging: rows of do and v; own value tiles of v_new and dv_new ------------------------------------------
#pragma unroll
    for (int j = 0; j < NRI / NW; ++j) {
        const int i = w + j * NW, m = i / (CH / RPI), r = (i % (CH / RPI)) * RPI + l / LPR;
        *reinterpret_cast<i32x4*>(&sTok[(m * CH + r) * VP + (l % LPR) * EPL]) = r < cp.len ? rows[j] : (i32x4){0, 0, 0, 0};
    }
    // v_new is not checkpointed by the scan: v_new_s = w_s S + u_s is rebuilt here from the checkpoint of S, which
    // is stored as exactly the operand this product needs (fragments of S^T), with the same bf16 operands and
    // fp32 accumulation as in the scan.  dv_new arrives as fragments of the transposed tiles (rows value, inner
    // token); one transposing product each gives the rows.
    Frag<T> uN[VTW][2];                                       // u of the own value tiles: rows token, inner value
#pragma unroll
    for (int j = 0; j < VTW; ++j) {
        f32x4 vn0 = zero4(), vn1 = zero4();
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            vn0 = mm(wf[0][kt], hv[j][kt], vn0);
            vn1 = mm(wf[1][kt], hv[j][kt], vn1);
        }
        uN[j][0] = transpose(ut[j][0], ident);
        uN[j][1] = transpose(ut[j][1], ident);
        vn0 += to_f32(uN[j][0]);
        vn1 += to_f32(uN[j][1]);
        T* dst = &sTok[c * VP + 16 * (vt0 + j) + 4 * g];
        st_frag(dst + 2 * CH * VP, to_frag<T>(vn0));
        st_frag(dst + 3 * CH * VP, to_frag<T>(vn1));
        st_frag(dst + 4 * CH * VP, transpose(yt[j][0], ident));
        st_frag(dst + 5 * CH * VP, transpose(yt[j][1], ident));
    }
    if (!EARLY) { own_kt_tiles(HC, hk); own_w_tiles(); }
    __syncthreads();                                           // (1) sTok, sScore, sKg complete
    auto tokf = [&](int m, int vt) __attribute__((always_inline)) { return ld_frag(&sTok[(m * CH + c) * VP + 16 * vt + 4 * g]); };

    Frag<T> aqkTf, aakTf[2];
    {
        f32x4 t[3] = {zero4(), zero4(), zero4()};
#pragma unroll
        for (int ww = 0; ww < NW; ++ww)
#pragma unroll
            for (int i = 0; i < 3; ++i) t[i] += *reinterpret_cast<const f32x4*>(sScore + ((ww * 3 + i) * 64 + l) * 4);
        if (HD) {
            // s of the own token (lane c), and beta, s of the four tokens this lane holds along the inner index
            f32x4 si = zero4();
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) {
                s_t += sRed[(ww * 3 + 0) * CH + c];
                si += *reinterpret_cast<const f32x4*>(sRed + (ww * 3 + 0) * CH + 4 * g);
            }
            const f32x4 bi = *reinterpret_cast<const f32x4*>(sRed + 1 * CH + 4 * g);
            const f32x4 x1 = t[1], x2 = t[2];
            t[1] = -bi * x1;
            t[2] = bi * bi * si * x1 - bi * x2;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {          // row j = c, inner i = 4g+i
            const int ii = 4 * g + i;
            if (!(c <= ii)) t[0][i] = 0.f;
            if (!(c < ii)) { t[1][i] = 0.f; t[2][i] = 0.f; }
        }
        aqkTf = to_frag<T>(t[0]);
        aakTf[0] = to_frag<T>(t[1]);
        aakTf[1] = to_frag<T>(t[2]);
    }

    // ---- own value tiles: products over the value dimension ------------------------------------------------------
    f32x4 dAqk = zero4(), dAqb[2] = {zero4(), zero4()}, dAak[2] = {zero4(), zero4()};
    f32x4 dAab[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
    f32x4 dv[VTW];
#pragma unroll
    for (int j = 0; j < VTW; ++j) {
        const int vt = vt0 + j;
        const Frag<T> doN = tokf(0, vt);
        const Frag<T> vN = tokf(1, vt);
        const Frag<T> vnN[2] = {tokf(2, vt), tokf(3, vt)};
        dAqk = mm(doN, vN, dAqk);
        dAqb[0] = mm(doN, vnN[0], dAqb[0]);
        dAqb[1] = mm(doN, vnN[1], dAqb[1]);
        const Frag<T> doT = transpose(doN, ident);
        Frag<T> dMf[2], dMTf[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            f32x4 x = mm(tmT[0][r], yt[j][0], zero4());
            x = mm(tmT[1][r], yt[j][1], x);
            dMf[r] = to_frag<T>(x);                       // dM_r   rows i, inner value
            f32x4 y = mm(yt[j][0], tmT[0][r], zero4());
            y = mm(yt[j][1], tmT[1][r], y);
            dMTf[r] = to_frag<T>(y);                      // dM_r^T rows value, inner i
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            dAak[r] = mm(dMf[r], vN, dAak[r]);
            dAab[r][0] = mm(dMf[r], uN[j][0], dAab[r][0]);
            dAab[r][1] = mm(dMf[r], uN[j][1], dAab[r][1]);
        }
        f32x4 x = mm(aqkTf, doT, zero4());
        x = mm(aakTf[0], dMTf[0], x);
        x = mm(aakTf[1], dMTf[1], x);
        dv[j] = x;                                        // rows token, inner value; kg dS is added at the end
    }

    // ---- own channel tiles, first pass: dw -> dag -> the w part of dA_ab -------------------------------------------
    Frag<T> Sf[KTW][VT];                                      // S of the own channel tiles: rows channel, inner value
    f32x4 dag[KTW][2];                                        // dag_r = sum_s (Tm^{s r})^T dw_s, rows token, inner channel
#pragma unroll
    for (int j = 0; j < KTW; ++j) {
        f32x4 dwT[2] = {zero4(), zero4()};                // rows channel, inner token
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            Sf[j][vt] = transpose(hk[j][vt], ident);
            dwT[0] = mm(Sf[j][vt], tokf(4, vt), dwT[0]);
            dwT[1] = mm(Sf[j][vt], tokf(5, vt), dwT[1]);
        }
        const Frag<T> dwTf[2] = {to_frag<T>(dwT[0]), to_frag<T>(dwT[1])};
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            dag[j][r] = mm(tmT[0][r], dwTf[0], zero4());
            dag[j][r] = mm(tmT[1][r], dwTf[1], dag[j][r]);
            const Frag<T> dagf = to_frag<T>(dag[j][r]);
            dAab[r][0] = mm(dagf, wk[0][j], dAab[r][0]);
            dAab[r][1] = mm(dagf, wk[1][j], dAab[r][1]);
        }
    }
    // tile indices: 0 A_qk, 1+s A_qb^s, 3+s A_ak^s, 5+2r+s A_ab^{r s}
    // Sum over the waves in two rounds (half the LDS of one round): the upper half of the waves leave their parts,
    // the lower half add them to their own and leave the sums.
    if (!EARLY) { own_kt_tile(DHC, dhk[0], 0); own_vt_tiles(DHC, dhv); load_b(); }
    {
        f32x4* const tiles[9] = {&dAqk, &dAqb[0], &dAqb[1], &dAak[0], &dAak[1], &dAab[0][0], &dAab[0][1], &dAab[1][0], &dAab[1][1]};
        float* const slot = sPart + (w % (NW / 2)) * 9 * 256;
        if (w >= NW / 2) {
#pragma unroll
            for (int i = 0; i < 9; ++i) *reinterpret_cast<f32x4*>(slot + (i * 64 + l) * 4) = *tiles[i];
        }
        __syncthreads();                                       // (2a)
        if (w < NW / 2) {
#pragma unroll
            for (int i = 0; i < 9; ++i) {
                f32x4* const q = reinterpret_cast<f32x4*>(slot + (i * 64 + l) * 4);
                *q = *q + *tiles[i];
            }
        }
    }
    __syncthreads();                                           // (2b) the parts of the nine tiles are complete
    // the waves share out the nine tiles: sum of the parts, causal mask, both orientations as fragments
#pragma unroll
    for (int t = 0; t < (9 + NW - 1) / NW; ++t) {
        const int idx = w + t * NW;
        if (idx < 9) {
            f32x4 x = zero4();
#pragma unroll
            for (int ww = 0; ww < NW / 2; ++ww) x += *reinterpret_cast<const f32x4*>(sPart + ((ww * 9 + idx) * 64 + l) * 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {      // row i = c, inner j = 4g+i; A_qk and A_qb keep the diagonal
                const int jj = 4 * g + i;
                if (idx < 3 ? !(jj <= c) : !(jj < c)) x[i] = 0.f;
            }
            const Frag<T> f = to_frag<T>(x);
            st_tile(sFin + idx * TILE, f);
            st_tile(sFin + (9 + idx) * TILE, transpose(f, ident));
        }
    }
    __syncthreads();                                           // (3) sFin complete; sPart may be overwritten (sOut)
    auto fin = [&](int idx) __attribute__((always_inline)) { return ld_tile(sFin + idx * TILE); };
    auto finT = [&](int idx) __attribute__((always_inline)) { return ld_tile(sFin + (9 + idx) * TILE); };
    // put(m, kt, f): tile f of gradient m (0 dq, 1 dk, 2/3 da, 4/5 db, 6 dgk) at channel tile kt of the staged rows
    auto put = [&](int m, int kt, Frag<T> f) __attribute__((always_inline)) {
        st_frag(reinterpret_cast<T*>(sOut + (m * CH + c) * L::OPK) + 16 * kt + 4 * g, f);
    };

    // ---- own value tiles: dv += kg dS over all channel tiles ------------------------------------------------------
#pragma unroll
    for (int j = 0; j < VTW; ++j) {
        f32x4 x = dv[j];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) x = mm(ld_tile(sKg + kt * TILE), dhv[j][kt], x);
        if (STAGE_OUT) st_frag(reinterpret_cast<T*>(sOut + 7 * CH * L::OPK + c * L::OPV) + 16 * (vt0 + j) + 4 * g, to_frag<T>(x));
        else if (rowok) st_frag(at(p.dv + vb, vo + 16 * (vt0 + j) * ES), to_frag<T>(x));
    }
    // ---- own channel tiles, second pass: state products, score backward, final gradients ---------------------------
    f32x4 dk_pre[(HD && !STAGE_OUT) ? KTW : 1], dg_pre[(HD && !STAGE_OUT) ? KTW : 1];
    float red[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KTW; ++j) {
        const int kt = kt0 + j;
        const f32x4 g4 = rg[j];
        const f32x4 gi = scan16_incl(g4);
        const f32x4 gl = bcast16(gi, CH - 1);
        const f32x4 edn = exp4<T>(gl - gi);
        const f32x4 k4 = to_f32(rk[j]);
        const f32x4 kg4 = k4 * edn;

        f32x4 dqg = zero4(), dkg = zero4(), dbg[2] = {zero4(), zero4()};
        float hh = 0.f;                                    // partial of sum_v S * dS for channel 16kt + c
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const Frag<T> dSf = transpose(dhk[j][vt], ident);
            dqg = mm(tokf(0, vt), Sf[j][vt], dqg);
            dkg = mm(tokf(1, vt), dSf, dkg);
            dbg[0] = mm(tokf(2, vt), dSf, dbg[0]);
            dbg[1] = mm(tokf(3, vt), dSf, dbg[1]);
            const f32x4 s4 = to_f32(Sf[j][vt]), d4 = to_f32(dSf);
            hh += s4[0] * d4[0] + s4[1] * d4[1] + s4[2] * d4[2] + s4[3] * d4[3];
        }
        if (!EARLY && KTW == 2 && j == 0) own_kt_tile(DHC, dhk[KTW - 1], 1);
        hh += __shfl_xor(hh, 16);
        hh += __shfl_xor(hh, 32);
        f32x4 hh4;
#pragma unroll
        for (int i = 0; i < 4; ++i) hh4[i] = __shfl(hh, 4 * g + i);

        // the factorised operands and decay factors of this channel tile, for the score backward
        const f32x4 ge = gi - g4;
        const f32x4 m = bcast16(gi, MID);
        const f32x4 eq = exp4<T>(gi - m), ek = exp4<T>(m - gi), ea = exp4<T>(ge - m);
        const f32x4 egi = exp4<T>(gi), ege = exp4<T>(ge);
        const f32x4 q4 = to_f32(rq[j]);
        const f32x4 a4[2] = {to_f32(a_of(0, j)), to_f32(a_of(1, j))};
        const f32x4 b4[2] = {to_f32(b_of(0, j)), to_f32(b_of(1, j))};
        const Frag<T> qh = to_frag<T>(q4 * eq * scale), kh = to_frag<T>(k4 * ek);
        const Frag<T> ah[2] = {to_frag<T>(a4[0] * ea), to_frag<T>(a4[1] * ea)};
        const Frag<T> bh[2] = {to_frag<T>(b4[0] * ek), to_frag<T>(b4[1] * ek)};
        const Frag<T> qhT = transpose(qh, ident), khT = transpose(kh, ident);
        const Frag<T> ahT[2] = {transpose(ah[0], ident), transpose(ah[1], ident)};
        const Frag<T> bhT[2] = {transpose(bh[0], ident), transpose(bh[1], ident)};
        const f32x4 bg4[2] = {b4[0] * edn, b4[1] * edn};
        f32x4 dqh = mm(fin(0), khT, zero4());
        dqh = mm(fin(1), bhT[0], dqh);
        dqh = mm(fin(2), bhT[1], dqh);
        f32x4 dkh = mm(finT(0), qhT, zero4());
        dkh = mm(finT(3), ahT[0], dkh);
        dkh = mm(finT(4), ahT[1], dkh);
        f32x4 dah[2], dbh[2];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            f32x4 x = mm(fin(3 + r), khT, zero4());
            x = mm(fin(5 + 2 * r), bhT[0], x);
            x = mm(fin(6 + 2 * r), bhT[1], x);
            dah[r] = x;
            f32x4 y = mm(finT(1 + r), qhT, zero4());          // here r plays the role of the b rank s
            y = mm(finT(5 + r), ahT[0], y);
            y = mm(finT(7 + r), ahT[1], y);
            dbh[r] = y;
        }
        const f32x4 dq = (dqh * eq + dqg * egi) * scale;
        const f32x4 dk = dkh * ek + dkg * edn;
        const f32x4 da[2] = {dah[0] * ea + dag[j][0] * ege, dah[1] * ea + dag[j][1] * ege};
        const f32x4 db[2] = {dbh[0] * ek + dbg[0] * edn, dbh[1] * ek + dbg[1] * edn};
        // The gradient of the log-decay sums, over token pairs (i, j) of the chunk, score-gradient times score with
        // opposite signs on the two tokens (Dgi: dependence through the inclusive decay sums, Dge: through the
        // exclusive ones); in the suffix sum below all pairs on one side of a token cancel, and they only do so if
        // both occurrences are the same number: the score part of each term therefore multiplies the factorised
        // operand as the products above saw it (rounded to the element type), not its exact value.
        const f32x4 st = dkg * kg4 + dbg[0] * bg4[0] + dbg[1] * bg4[1];      // the state-path part of k and b
        const f32x4 Dge = dah[0] * to_f32(ah[0]) + dah[1] * to_f32(ah[1]) + (dag[j][0] * a4[0] + dag[j][1] * a4[1]) * ege;
        const f32x4 Dgi = dqh * to_f32(qh) + dqg * (q4 * egi * scale) - dkh * to_f32(kh)
                          - dbh[0] * to_f32(bh[0]) - dbh[1] * to_f32(bh[1]) - st;
        const f32x4 dgl = exp4<T>(gl) * hh4 + sum16(st);
        const f32x4 dg = rscan16_incl(Dgi + Dge) - Dge + dgl;
        if (HD) {
            // backward of the parameterisation, the part that needs no sum over channels; what does (through s, and
            // dbeta itself) waits for the sums r1 = sum k da_1, r2 = sum k da_2, r3 = sum k f da_2 of all the waves
            const f32x4 f4 = exp4<T>(g4);
            const f32x4 dkp = dk - da[0] * beta_t + da[1] * ((beta_t * s_t - f4) * beta_t) + db[0] * f4 + db[1];
            const f32x4 dgp = dg + (db[0] - da[1] * beta_t) * k4 * f4;
            if (STAGE_OUT) {       // kept, per lane, in the rows of the staging area that da and db do not use here
                *reinterpret_cast<f32x4*>(sOut + 2 * CH * L::OPK + ((w * KTW + j) * 2 + 0) * 1024 + l * 16) = dkp;
                *reinterpret_cast<f32x4*>(sOut + 2 * CH * L::OPK + ((w * KTW + j) * 2 + 1) * 1024 + l * 16) = dgp;
            } else {
                dk_pre[j] = dkp;
                dg_pre[j] = dgp;
            }
            const f32x4 t1 = k4 * da[0], t2 = k4 * da[1], t3 = t2 * f4;
            red[0] += t1[0] + t1[1] + t1[2] + t1[3];
            red[1] += t2[0] + t2[1] + t2[2] + t2[3];
            red[2] += t3[0] + t3[1] + t3[2] + t3[3];
            if (STAGE_OUT) put(0, kt, to_frag<T>(dq));
            else if (rowok) st_frag(at(p.dq + qb, qo + 16 * kt * ES), to_frag<T>(dq));
        } else if (STAGE_OUT) {
            put(0, kt, to_frag<T>(dq));
            put(1, kt, to_frag<T>(dk));
            put(2, kt, to_frag<T>(da[0]));
            put(3, kt, to_frag<T>(da[1]));
            put(4, kt, to_frag<T>(db[0]));
            put(5, kt, to_frag<T>(db[1]));
            if (!GKF32) put(6, kt, to_frag<T>(dg));
            else if (rowok) st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
        } else if (rowok) {
            st_frag(at(p.dq + qb, qo + 16 * kt * ES), to_frag<T>(dq));
            st_frag(at(p.dk + qb, qo + 16 * kt * ES), to_frag<T>(dk));
            st_frag(at(p.da + ab, ao0 + 16 * kt * ES), to_frag<T>(da[0]));
            st_frag(at(p.da + ab, ao1 + 16 * kt * ES), to_frag<T>(da[1]));
            st_frag(at(p.db + ab, ao0 + 16 * kt * ES), to_frag<T>(db[0]));
            st_frag(at(p.db + ab, ao1 + 16 * kt * ES), to_frag<T>(db[1]));
            st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
        }
        // the large shapes are at the limit of the register file: keep the two channel tiles from being interleaved
        if (!EARLY) __builtin_amdgcn_sched_barrier(0);
    }
    if (HD) {
        // sums over all channels, per token: within the wave over the four lane groups, then over the waves through LDS
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            red[i] = sum_groups(red[i]);
            if (g == 0) sRed[(w * 3 + i) * CH + c] = red[i];
        }
        __syncthreads();                                       // (3b) the sums of all waves are there
        float r1 = 0.f, r2 = 0.f, r3 = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) {
            r1 += sRed[(ww * 3 + 0) * CH + c];
            r2 += sRed[(ww * 3 + 1) * CH + c];
            r3 += sRed[(ww * 3 + 2) * CH + c];
        }
        // a_2 depends on every channel through s: ds = beta^2 r2, and s = sum k^2 f
        const float ds = beta_t * beta_t * r2;
#pragma unroll
        for (int j = 0; j < KTW; ++j) {
            const int kt = kt0 + j;
            const f32x4 k4 = to_f32(rk[j]), kf = k4 * exp4<T>(rg[j]);
            const f32x4 dkp = STAGE_OUT ? *reinterpret_cast<const f32x4*>(sOut + 2 * CH * L::OPK + ((w * KTW + j) * 2 + 0) * 1024 + l * 16) : dk_pre[j];
            const f32x4 dgp = STAGE_OUT ? *reinterpret_cast<const f32x4*>(sOut + 2 * CH * L::OPK + ((w * KTW + j) * 2 + 1) * 1024 + l * 16) : dg_pre[j];
            const f32x4 dk = dkp + kf * (2.f * ds);
            const f32x4 dg = dgp + kf * k4 * ds;
            if (STAGE_OUT) {
                put(1, kt, to_frag<T>(dk));
                if (!GKF32) put(6, kt, to_frag<T>(dg));
                else if (rowok) st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
            } else if (rowok) {
                st_frag(at(p.dk + qb, qo + 16 * kt * ES), to_frag<T>(dk));
                st_gk4<GKF32>(dgkp + go + 16 * kt * GS, 0, dg);
            }
        }
        // dbeta = sum_c da_1 (-k) + da_2 k (2 beta s - f)
        if (w == 0 && g == 0 && rowok) st_elem(p.dbeta + (cp.tok0 + c) * H + h, -r1 + 2.f * beta_t * s_t * r2 - r3);
    }
    if (STAGE_OUT) {
        __syncthreads();                                       // (4) the staged rows are complete
        // whole rows, 16 bytes a lane; the waves take turns over the instructions
        constexpr int LRK = K * (int)ES / 16, RPK = 64 / LRK, NUK = CH / RPK;   // lanes per row, rows per instruction, instructions per tensor
        constexpr int LRV = V * (int)ES / 16, RPV = 64 / LRV, NUV = CH / RPV;
        // gradients that leave through the staged rows: dq, dk, da (2), db (2), dgk; with the HDLA parameterisation
        // dq, dk, dgk; dgk goes out directly when it is fp32 next to 2-byte inputs
        constexpr int NKT = HD ? (GKF32 ? 2 : 3) : (GKF32 ? 6 : 7), NU = NKT * NUK + NUV;
        const uint32_t qpitch = (uint32_t)(H * K) * ES, apitch = qpitch * RANK;
#pragma unroll
        for (int t = 0; t < (NU + NW - 1) / NW; ++t) {
            const int u = w + t * NW;
            if (u < NKT * NUK) {
                const int mi = u / NUK, m = (HD && mi == 2) ? 6 : mi, r = (u % NUK) * RPK + l / LRK, e = (l % LRK) * 16;
                char* base = reinterpret_cast<char*>(m == 0 ? p.dq + qb : m == 1 ? p.dk + qb : m < 4 ? p.da + ab : m < 6 ? p.db + ab : reinterpret_cast<T*>(dgkp));
                const uint32_t pitch = (m < 2 || m == 6) ? qpitch : apitch, off = (m == 3 || m == 5) ? qpitch : 0;
                const i32x4 x = *reinterpret_cast<const i32x4*>(sOut + (m * CH + r) * L::OPK + e);
                if (r < cp.len) *reinterpret_cast<i32x4*>(base + (uint32_t)r * pitch + off + e) = x;
            } else if (u < NU) {
                const int r = (u - NKT * NUK) * RPV + l / LRV, e = (l % LRV) * 16;
                const i32x4 x = *reinterpret_cast<const i32x4*>(sOut + 7 * CH * L::OPK + r * L::OPV + e);
                if (r < cp.len) *reinterpret_cast<i32x4*>(reinterpret_cast<char*>(p.dv + vb) + (uint32_t)r * (uint32_t)(H * V) * ES + e) = x;
            }
        }
    }
}

template <typename T, int K, int V, bool HD>
static hipError_t launch_chunk_grad_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.st.nch * a.H), block(64 * NW);
    constexpr bool kAlwaysF32 = sizeof(T) == 4;
    if (kAlwaysF32 || a.gk_f32) hipLaunchKernelGGL((chunk_grad_kernel<T, true, K, V, HD>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((chunk_grad_kernel<T, kAlwaysF32, K, V, HD>), grid, block, 0, stream, a);
    return hipGetLastError();
}

template <typename T, bool HD>
static hipError_t launch_chunk_grad_hd(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_chunk_grad_kv<T, 64, 64, HD>(a, stream);
    if (K == 128 && V == 128) return launch_chunk_grad_kv<T, 128, 128, HD>(a, stream);
    if (K == 64 && V == 128) return launch_chunk_grad_kv<T, 64, 128, HD>(a, stream);
    if (K == 128 && V == 64) return launch_chunk_grad_kv<T, 128, 64, HD>(a, stream);
    return hipErrorInvalidValue;
}

template <typename T>
hipError_t launch_chunk_grad(const ChunkArgs<T>& a, int K, int V, hipStream_t stream) {
    return a.beta ? launch_chunk_grad_hd<T, true>(a, K, V, stream) : launch_chunk_grad_hd<T, false>(a, K, V, stream);
}
template hipError_t launch_chunk_grad<bf16>(const ChunkArgs<bf16>&, int, int, hipStream_t);
template hipError_t launch_chunk_grad<float>(const ChunkArgs<float>&, int, int, hipStream_t);

}  // namespace hdla
