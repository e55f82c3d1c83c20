// prep kernel: everything of a 16-token chunk that does not depend on the recurrent state.
//
// Replaces, for one (chunk, head) per workgroup, the reference's chunk-local cumsum (fla chunk_rwkv6_fwd_cumsum,
// called at HRDPLR/hrdplr.py:44), the two score kernels (HRDPLR/fwd_triton.py:22-290 and :305-514), the
// triangular inverse (HRDPLR/fwd_triton.py:601-667) and the WY kernel (HRDPLR/fwd_triton.py:685-790).
// The four score matrices never reach HBM: they are MFMA accumulators, (I - A_ab)^-1 is solved in LDS, and
// w, u and the gated copies are written once, in the fragment order the state scans read them in.
//
// A wave handles 64 channels: K = 64 is one wave per (chunk, head); K = 128 is a workgroup of two, each with its
// half of the channel tiles and of the value tiles.  The score tiles are sums over channels: the two exchange
// their parts through LDS and each then solves the (small) triangular system for itself.  One wave with all 128
// channels needs the whole register file, and at one wave per SIMD nothing hides its memory round trips.
#include "hdla_common.cuh"
#include "hdla_launch.h"

namespace hdla {

constexpr int LDP = 36;   // padded row length of the 32x32 LDS matrices (keeps 16-byte row alignment)

// MODE: what the kernel leaves in the workspace -- PREP_FWD: what the forward pass's scan reads (which also forms the
// output); PREP_BWD: what the two scans of the backward pass and the chunk_grad kernels read; PREP_KEEP: both, for a
// forward pass whose workspace the backward pass will use instead of running this kernel again.
enum PrepMode { PREP_FWD = 0, PREP_BWD = 1, PREP_KEEP = 2 };
template <typename T, bool GKF32, int K, int V, int MODE, bool HD>
__global__ __launch_bounds__(K) __attribute__((amdgpu_waves_per_eu(2, 2))) void prep_kernel(ChunkArgs<T> p) {
    constexpr bool BWD = MODE == PREP_BWD;                // neither the output's score tiles nor qg are needed
    constexpr bool WB = MODE != PREP_FWD;                 // the backward pass's extras are
    constexpr int NWP = K / 64;                       // waves per (chunk, head)
    constexpr int KTW = 4, VT = V / 16, VTW = VT / NWP, KT2 = K / 32;
    constexpr int SAS = blk_fwd(K, sizeof(T), !BWD).SIZE / (int)sizeof(T);   // elements between (chunk, head) slots
    constexpr int SBS = blk_bwd(K, sizeof(T)).SIZE / (int)sizeof(T);
    __shared__ __attribute__((aligned(16))) float sNw[NWP][32 * LDP];   // A_ab, rank-major (one copy per wave)
    __shared__ __attribute__((aligned(16))) float sTw[NWP][32 * LDP];   // (I - A_ab)^-1
    constexpr int NPART = BWD ? 8 : 9;                                    // score tiles that are summed over the waves
    __shared__ __attribute__((aligned(16))) float sPart[NWP > 1 ? NWP * NPART * 256 : 4];
    __shared__ int sStrong[NWP];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float* const sN = sNw[w];
    float* const sT = sTw[w];
    const int kt0 = w * KTW, vt0 = w * VTW;                              // first own channel tile / value tile

    // Which of the two indices runs fastest over the workgroups decides which rows of the [token][head][channel]
    // tensors the workgroups resident at one time touch.  Measured: with rows of 4 KiB and more, neighbouring
    // workgroups should be the heads of one chunk (together they read whole rows; chunk-fastest, all of them would
    // touch the same few hundred bytes of every row, a fraction of the HBM channels); with shorter rows the chunks
    // of one head, whose workspace records are contiguous.
    const bool head_fastest = (uint32_t)(p.H * K) * sizeof(T) >= 4096;
    const int cid = head_fastest ? blockIdx.x / p.H : blockIdx.x % p.st.nch;
    const int h = head_fastest ? blockIdx.x % p.H : blockIdx.x / p.st.nch;
    ChunkPos cp;
    if (!locate_chunk(p.st, cid, cp)) return;
    const int l = lane_id(), g = l >> 4, c = l & 15;
    const int H = p.H;
    const bool rowok = c < cp.len;
    const int64_t tok = cp.tok0 + min(c, cp.len - 1);   // rows past the end alias the last valid row, masked by rowok
    const int64_t qoff = (tok * H + h) * K + 4 * g;                 // + 16*kt
    const int64_t aoff0 = ((tok * RANK + 0) * H + h) * K + 4 * g;
    const int64_t aoff1 = ((tok * RANK + 1) * H + h) * K + 4 * g;
    const int64_t voff = (tok * H + h) * V + 4 * g;
    const int64_t chw = (int64_t)h * p.st.nch + cid;                // chunk-head slot in the workspace
    const float scale = p.scale;

    // ---- phase A: cumulative decays and the score tiles (rows i, inner j) -----------------------------------
    f32x4 gi[KTW], ge[KTW];
    f32x4 aqk = zero4(), aqb[2] = {zero4(), zero4()}, aak[2] = {zero4(), zero4()};
    f32x4 aab[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
    // the inputs of the chunk stay in registers (as loaded) for the second use in phase C: the working set of the
    // resident waves is larger than the L2, so a second load would come from HBM again
    Frag<T> rq[KTW], rk[KTW], ra[2][KTW], rb[2][KTW];       // own channel tiles; index kt below is local, kt0 + kt global
    // v is used last (phase D) but requested first: the barriers in between would otherwise keep its loads, and a
    // full round trip to HBM, behind everything else
    Frag<T> rv[VTW];
#pragma unroll
    for (int vt = 0; vt < VTW; ++vt) rv[vt] = ld_frag_sel(p.v + voff + 16 * (vt0 + vt), rowok);
    // HDLA parameterisation: a_1 = -beta k, a_2 = beta k (beta s - f), b_1 = f k, b_2 = k with f = exp(gk) and
    // s = sum over ALL channels of k^2 f (a wave reads the other waves' channels of k and gk for it as well)
    float beta_t = 0.f, s_t = 0.f;
    if (HD) {
        beta_t = rowok ? ld_elem(p.beta + tok * H + h) : 0.f;
#pragma unroll
        for (int kt = 0; kt < K / 16; ++kt) {
            const f32x4 g4 = ld_gk4<GKF32>(p.gk, qoff + 16 * kt, rowok);
            const f32x4 k4 = to_f32(ld_frag_sel(p.k + qoff + 16 * kt, rowok));
            const f32x4 kf = k4 * k4 * exp4<T>(g4);
            s_t += kf[0] + kf[1] + kf[2] + kf[3];
        }
        s_t += __shfl_xor(s_t, 16);
        s_t += __shfl_xor(s_t, 32);
    }
#pragma unroll
    for (int kt = 0; kt < KTW; ++kt) {
        const int ko = 16 * (kt0 + kt);
        const f32x4 g4 = ld_gk4<GKF32>(p.gk, qoff + ko, rowok);
        rq[kt] = ld_frag_sel(p.q + qoff + ko, rowok);
        rk[kt] = ld_frag_sel(p.k + qoff + ko, rowok);
        if (HD) {
            const f32x4 kk = to_f32(rk[kt]), f4 = exp4<T>(g4);
            ra[0][kt] = to_frag<T>(kk * (-beta_t));
            ra[1][kt] = to_frag<T>(kk * ((beta_t * s_t - f4) * beta_t));
            rb[0][kt] = to_frag<T>(f4 * kk);
            rb[1][kt] = rk[kt];
        } else {
            ra[0][kt] = ld_frag_sel(p.a + aoff0 + ko, rowok);
            ra[1][kt] = ld_frag_sel(p.a + aoff1 + ko, rowok);
            rb[0][kt] = ld_frag_sel(p.b + aoff0 + ko, rowok);
            rb[1][kt] = ld_frag_sel(p.b + aoff1 + ko, rowok);
        }
        gi[kt] = scan16_incl(g4);
        ge[kt] = gi[kt] - g4;
        // Every score is a dense product of operands decayed relative to the middle of the chunk: exp(gi_i - gi_j) =
        // exp(gi_i - m) exp(m - gi_j) with m = gi of token MID.  That is done here for every chunk, tile by tile as the
        // inputs arrive; it is only valid while the exponents stay within +-SAFE_RANGE, which is checked afterwards.
        const f32x4 m = bcast16<MID>(gi[kt]);
        const f32x4 eq = exp4<T>(gi[kt] - m), ek = exp4<T>(m - gi[kt]), ea = exp4<T>(ge[kt] - m);
        const f32x4 q4 = to_f32(rq[kt]), k4 = to_f32(rk[kt]);
        const f32x4 a0 = to_f32(ra[0][kt]), a1 = to_f32(ra[1][kt]), b0 = to_f32(rb[0][kt]), b1 = to_f32(rb[1][kt]);
        Split<T> qh, kh, ah[2], bh[2];
        split(q4 * eq * scale, qh);
        split(k4 * ek, kh);
        split(a0 * ea, ah[0]);
        split(a1 * ea, ah[1]);
        split(b0 * ek, bh[0]);
        split(b1 * ek, bh[1]);
        aqk = mm3(qh, kh, aqk);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            aqb[s] = mm3(qh, bh[s], aqb[s]);
            aak[s] = mm3(ah[s], kh, aak[s]);
#pragma unroll
            for (int r = 0; r < 2; ++r) aab[r][s] = mm3(ah[r], bh[s], aab[r][s]);
        }
    }
    // Each wave decides for its own channels (the parts of the score tiles add up whichever way they were formed); the
    // backward pass records the decision per (chunk, head) for the chunk_grad kernels.  Where a channel decays too
    // strongly for the single centre, what was accumulated above may hold infinities: it is thrown away and the tiles
    // are formed again by passes whose exponents cannot overflow (see DecayPass).
    const bool strong = strong_decay(gi, ge);
    if (WB && l == 0) {
        if (NWP == 1) p.ws.STRONG[chw] = strong;
        else sStrong[w] = strong;
    }
    if (strong) {
        aqk = zero4();
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            aqb[s] = zero4(); aak[s] = zero4(); aab[0][s] = zero4(); aab[1][s] = zero4();
        }
#pragma unroll 1
        for (int ps = 0; ps < DecayPass::COUNT; ++ps) {
            const DecayPass dp(ps, c);
#pragma unroll
            for (int kt = 0; kt < KTW; ++kt) {
                f32x4 eq, ek, ea;
                dp.factors<T>(gi[kt], ge[kt], eq, ek, ea);
                // the same products as above, one operand at a time with the scheduler kept from interleaving them: this
                // path is rare and must not cost the common one registers
                // (pin(): the conversions of the inputs do not depend on the pass, and hoisted out of the pass loop they
                // would all be live across it)
                pin(rk[kt]); pin(rq[kt]); pin(ra[0][kt]); pin(ra[1][kt]); pin(rb[0][kt]); pin(rb[1][kt]);
                Split<T> qh, kh, bh[2];
                split(to_f32(rk[kt]) * ek, kh);
                split(to_f32(rq[kt]) * eq * scale, qh);
                aqk = mm3(qh, kh, aqk);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    split(to_f32(rb[s][kt]) * ek, bh[s]);
                    aqb[s] = mm3(qh, bh[s], aqb[s]);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int r = 0; r < 2; ++r) {
                    Split<T> ah;
                    split(to_f32(ra[r][kt]) * ea, ah);
                    aak[r] = mm3(ah, kh, aak[r]);
                    aab[r][0] = mm3(ah, bh[0], aab[r][0]);
                    aab[r][1] = mm3(ah, bh[1], aab[r][1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
    if (NWP > 1) {
        // sums over all channels: every wave leaves its parts in LDS and adds the others'
        f32x4* const tiles[9] = {&aak[0], &aak[1], &aab[0][0], &aab[0][1], &aab[1][0], &aab[1][1],
                                 &aqb[0], &aqb[1], &aqk};
#pragma unroll
        for (int i = 0; i < NPART; ++i) *reinterpret_cast<f32x4*>(&sPart[((w * NPART + i) * 64 + l) * 4]) = *tiles[i];
        __syncthreads();
#pragma unroll
        for (int ww = 1; ww < NWP; ++ww)
#pragma unroll
            for (int i = 0; i < NPART; ++i)
                *tiles[i] += *reinterpret_cast<const f32x4*>(&sPart[((((w + ww) % NWP) * NPART + i) * 64 + l) * 4]);
        if (WB && w == 0 && l == 0) {
            int any = 0;
#pragma unroll
            for (int ww = 0; ww < NWP; ++ww) any |= sStrong[ww];
            p.ws.STRONG[chw] = any;
        }
    }
    // causal masks: lane (g,c) reg i is entry (row c, inner 4g+i)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = 4 * g + i;
        const bool le = j <= c, lt = j < c;
        if (!le) { aqk[i] = 0.f; aqb[0][i] = 0.f; aqb[1][i] = 0.f; }
        if (!lt) { aak[0][i] = 0.f; aak[1][i] = 0.f; aab[0][0][i] = 0.f; aab[0][1][i] = 0.f; aab[1][0][i] = 0.f; aab[1][1][i] = 0.f; }
    }
    if (w == 0) {
        if (!BWD) {
            st_tile(p.ws.AQK + chw * SAS, to_frag<T>(aqk));
            st_pair2(p.ws.AQB + chw * SAS, to_frag<T>(aqb[0]), to_frag<T>(aqb[1]));
        }
        if (BWD || WB) {
            // the other orientation is the rounded tile turned (a product with the identity: exact), in every mode, so
            // that a backward pass finds the same bytes whether it recomputes them or reads what a forward pass kept
            const Frag<T> id = ident_frag<T>();
            st_pair2(p.ws.AQBT + chw * SBS, transpose(to_frag<T>(aqb[0]), id), transpose(to_frag<T>(aqb[1]), id));
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int s = 0; s < 2; ++s)
            *reinterpret_cast<f32x4*>(&sN[(16 * r + c) * LDP + 16 * s + 4 * g]) = aab[r][s];
    __syncthreads();

    // ---- phase B: (I - A_ab)^-1 -----------------------------------------------------------------------------------
    // In token halves, L = tokens 0..7 and H = 8..15 (both ranks: 16 rows each):
    //   (I - A)^-1 = [[T_LL, 0], [T_HL, T_HH]],  T_LL = (I - A_LL)^-1,  T_HH = (I - A_HH)^-1,  T_HL = T_HH A_HL T_LL.
    // The diagonal blocks by forward substitution over tokens, in registers, both at once: lane (r, half, column) builds
    // one column of the rows (r, i) of its half, one token per step, the entries of the other rank's rows coming from the
    // lane 32 positions away (eight steps and a quarter of the dependent multiply-adds of one substitution over all
    // sixteen tokens).  The block below the diagonal is two 16 x 16 x 16 products, in split operands like the score
    // products for 2-byte elements (the error of fp32 products), in fp32 products otherwise.
    {
        const int r = l >> 5, hf = (l >> 4) & 1, sc = (l >> 3) & 1, jc = l & 7;
        const int col = 16 * sc + 8 * hf + jc;
        float x[8], y[8];                        // own rows (r, j) and the partner's rows (1-r, j) of column col
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float* nrow = &sN[(16 * r + 8 * hf + i) * LDP + 8 * hf];
            float acc0 = (sc == r && jc == i) ? 1.f : 0.f, acc1 = 0.f;
#pragma unroll
            for (int j4 = 0; j4 < (i + 3) / 4; ++j4) {
                const f32x4 co = *reinterpret_cast<const f32x4*>(nrow + 16 * r + 4 * j4);         // own rank block
                const f32x4 cx = *reinterpret_cast<const f32x4*>(nrow + 16 * (1 - r) + 4 * j4);   // other rank block
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
            sT[(16 * r + 8 * hf + i) * LDP + col] = x[i];
            if (hf == 0) sT[(16 * r + i) * LDP + col + 8] = 0.f;      // rows of L, columns of H: zero
        }
        // (the wave reads below what its other lanes wrote above: LDS accesses of one wave complete in order)
        // 16 x 16 matrices in (rank, token of the half) order: row c = 8 rank + token, inner 4g .. 4g+3 likewise
        const int rr = c >> 3, ii = c & 7, ss = g >> 1, j0 = 4 * (g & 1);
        const f32x4 ahl = *reinterpret_cast<const f32x4*>(&sN[(16 * rr + 8 + ii) * LDP + 16 * ss + j0]);
        const f32x4 thh = *reinterpret_cast<const f32x4*>(&sT[(16 * rr + 8 + ii) * LDP + 16 * ss + 8 + j0]);
        f32x4 tllT;                              // T_LL^T: row c is column c of T_LL
#pragma unroll
        for (int e = 0; e < 4; ++e) tllT[e] = sT[(16 * ss + j0 + e) * LDP + 16 * rr + ii];
        Split<T> pa, pb;
        split(tllT, pa);
        split(ahl, pb);
        const f32x4 xT = mm3(pa, pb, zero4());   // (A_HL T_LL)^T = T_LL^T A_HL^T
        split(thh, pa);
        split(xT, pb);
        const f32x4 thl = mm3(pa, pb, zero4());  // T_HH (A_HL T_LL)
        *reinterpret_cast<f32x4*>(&sT[(16 * rr + 8 + ii) * LDP + 16 * ss + j0]) = thl;
        __syncthreads();
    }
    Frag<T> tm[2][2];   // F(Tm^{s s'}): rows i, inner j
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
            tm[s][s2] = to_frag<T>(*reinterpret_cast<const f32x4*>(&sT[(16 * s + c) * LDP + 16 * s2 + 4 * g]));
    const Frag<T> ident = ident_frag<T>();
    if (WB && w == NWP - 1) {
        // for the chunk_grad kernel: the four blocks transposed, as fragments (two tile pairs), ready to load
        T* tmw = p.ws.TM + chw * 1024;
#pragma unroll
        for (int s = 0; s < 2; ++s) st_pair2(tmw + s * PAIR, transpose(tm[s][0], ident), transpose(tm[s][1], ident));
    }

    // ---- phase C: w = Tm ag and the gated copies, two channel tiles (one stored pair) at a time -----------------
#pragma unroll
    for (int kpl = 0; kpl < KTW / 2; ++kpl) {
        const int kp = kt0 / 2 + kpl;                         // stored pair
        Frag<T> fw[2][2], fkgT[2], fbgT[2][2], fqg[2], fqgT[2];   // [..][tile of the pair]
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int kt = 2 * kpl + e;
            const f32x4 gl = bcast16<CH - 1>(gi[kt]);
            const f32x4 egi = exp4<T>(gi[kt]), ege = exp4<T>(ge[kt]), edn = exp4<T>(gl - gi[kt]);
            const Frag<T> agT[2] = {transpose(to_frag<T>(to_f32(ra[0][kt]) * ege), ident),
                                    transpose(to_frag<T>(to_f32(ra[1][kt]) * ege), ident)};
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                f32x4 w = mm(tm[s][0], agT[0], zero4());
                w = mm(tm[s][1], agT[1], w);
                fw[s][e] = to_frag<T>(w);
            }
            fqg[e] = to_frag<T>(to_f32(rq[kt]) * egi * scale);
            const Frag<T> kg = to_frag<T>(to_f32(rk[kt]) * edn);
            fkgT[e] = transpose(kg, ident);
            fbgT[0][e] = transpose(to_frag<T>(to_f32(rb[0][kt]) * edn), ident);
            fbgT[1][e] = transpose(to_frag<T>(to_f32(rb[1][kt]) * edn), ident);
            if (WB) fqgT[e] = transpose(fqg[e], ident);
            if (c == 0) {
                const f32x4 egl = exp4<T>(gl);
                *reinterpret_cast<f32x4*>(p.ws.EGL + chw * (SAS * (int)sizeof(T) / 4) + 16 * (kt0 + kt) + 4 * g) = egl;
            }
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            st_pair2(p.ws.W + chw * SAS + (s * KT2 + kp) * PAIR, fw[s][0], fw[s][1]);
            st_pair2(p.ws.BGT + chw * SAS + (s * KT2 + kp) * PAIR, fbgT[s][0], fbgT[s][1]);
        }
        st_pair2(p.ws.KGT + chw * SAS + kp * PAIR, fkgT[0], fkgT[1]);
        if (!BWD) st_pair2(p.ws.QG + chw * SAS + kp * PAIR, fqg[0], fqg[1]);
        if (WB) st_pair2(p.ws.QGT + chw * SBS + kp * PAIR, fqgT[0], fqgT[1]);
    }

    // ---- phase D: u = Tm (A_ak v), kept transposed (rows value, inner token) ---------------------------------
    const Frag<T> aakf[2] = {to_frag<T>(aak[0]), to_frag<T>(aak[1])};
#pragma unroll
    for (int vl = 0; vl < VTW; ++vl) {
        const int vt = vt0 + vl;
        const Frag<T> vT = transpose(rv[vl], ident);
        st_tile(p.ws.VTT + (chw * VT + vt) * TILE, vT);
        const Frag<T> mT[2] = {to_frag<T>(mm(vT, aakf[0], zero4())), to_frag<T>(mm(vT, aakf[1], zero4()))};
        Frag<T> fu[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            f32x4 uT = mm(mT[0], tm[s][0], zero4());
            uT = mm(mT[1], tm[s][1], uT);
            fu[s] = to_frag<T>(uT);
        }
        st_pair2(p.ws.UT + (chw * VT + vt) * PAIR, fu[0], fu[1]);
    }
}

// ---- chunk table for packed variable-length batches ----------------------------------------------------------
constexpr int ORDER_MAX_N = 2048;      // beyond this many sequences they are taken as they come (ranking is quadratic)
constexpr int TABLE_THREADS = 256;
// Workgroup 0 builds the table; with at most ORDER_MAX_N sequences, workgroups 1 .. ceil(N / 256) rank the sequences by
// their chunk counts, one sequence a thread (they form the counts from cu themselves, so they wait for nobody).
__global__ __launch_bounds__(TABLE_THREADS) void build_chunk_table_kernel(const int64_t* cu, int N, int T, int nch, int32_t* chunk_off,
                                                                          int32_t* chunk_seq) {
    constexpr int LONG_SEQ = 64, LONG_LIST = 512;
    __shared__ long long strip[2][TABLE_THREADS];
    __shared__ __attribute__((aligned(16))) int32_t len[ORDER_MAX_N];
    __shared__ int n_long, long_seq[LONG_LIST], long_c0[LONG_LIST], long_c1[LONG_LIST];
    const int t = threadIdx.x;
    auto chunks_of = [&](int n) {
        int64_t bos, eos;
        packed_bounds(cu, n, T, bos, eos);
        return (long long)((eos - bos + CH - 1) / CH);
    };
    int32_t* order = chunk_off + N + 1;
    if (blockIdx.x > 0) {
        // order[r] = the sequence with the r-th most chunks (ties by index): the scans start their workgroups in this
        // order, so that when there are more workgroups than compute units the long sequences are not the ones that
        // wait.  All counts go to LDS (entries past N hold -1 and rank behind everything); a thread reads them four at
        // a time against its own.
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        for (int n = t; n < ORDER_MAX_N; n += TABLE_THREADS) len[n] = n < N ? (int)min(chunks_of(n), (long long)0x7fffffff) : -1;
        __syncthreads();
        const int n = ((int)blockIdx.x - 1) * TABLE_THREADS + t;
        if (n >= N) return;
        const int mine = len[n];
        int r = 0;
        for (int m = 0; m < N; m += 4) {
            const i32x4 lm = *reinterpret_cast<const i32x4*>(&len[m]);
#pragma unroll
            for (int j = 0; j < 4; ++j) r += (lm[j] > mine || (lm[j] == mine && m + j < n)) ? 1 : 0;
        }
        order[r] = n;
        return;
    }
    // chunk_off = exclusive prefix sum of the sequences' chunk counts: every thread sums a strip of consecutive
    // sequences, the strip sums are scanned in LDS, and the strips are walked a second time.
    const int per = (N + TABLE_THREADS - 1) / TABLE_THREADS;
    const int n0 = min(t * per, N), n1 = min(n0 + per, N);
    long long own = 0;
#pragma unroll 8
    for (int n = n0; n < n1; ++n) own += chunks_of(n);
    strip[0][t] = own;
    if (t == 0) n_long = 0;
    __syncthreads();
    int cur = 0;
    for (int d = 1; d < TABLE_THREADS; d <<= 1) {         // inclusive scan, one doubling step per round
        strip[cur ^ 1][t] = strip[cur][t] + (t >= d ? strip[cur][t - d] : 0);
        cur ^= 1;
        __syncthreads();
    }
    // chunk_off, and chunk_seq: a thread writes the entries of its own strip's sequences; sequences of more than
    // LONG_SEQ chunks are put on a list and written by the whole workgroup afterwards (a thread that finds the list
    // full writes its own).  Offsets never go beyond the slots the workspace has (cannot happen for a non-decreasing
    // table that ends at T).
    long long acc = strip[cur][t] - own;
    for (int n = n0; n < n1; ++n) {
        const long long nx = acc + chunks_of(n);
        const int c0 = (int)min(acc, (long long)nch), c1 = (int)min(nx, (long long)nch);
        acc = nx;
        chunk_off[n] = c0;
        int slot = LONG_LIST;
        if (c1 - c0 > LONG_SEQ) slot = atomicAdd(&n_long, 1);
        if (slot < LONG_LIST) { long_seq[slot] = n; long_c0[slot] = c0; long_c1[slot] = c1; }
        else for (int cid = c0; cid < c1; ++cid) chunk_seq[cid] = n;
    }
    if (t == 0) chunk_off[N] = (int)min(strip[cur][TABLE_THREADS - 1], (long long)nch);
    __syncthreads();
    const int nl = min(n_long, LONG_LIST);
    for (int i = 0; i < nl; ++i)
        for (int cid = long_c0[i] + t; cid < long_c1[i]; cid += TABLE_THREADS) chunk_seq[cid] = long_seq[i];
    if (N > ORDER_MAX_N)                                  // too many to rank: as they come
        for (int n = t; n < N; n += TABLE_THREADS) order[n] = n;
}

template <typename T, int K, int V, bool HD>
static hipError_t launch_prep_kv(const ChunkArgs<T>& a, int mode, hipStream_t stream) {
    dim3 grid(a.st.nch * a.H), block(K);
    constexpr bool kAlwaysF32 = sizeof(T) == 4;
    const bool gkf32 = kAlwaysF32 || a.gk_f32;
#define HDLA_PREP_LAUNCH(GK, MODE) hipLaunchKernelGGL((prep_kernel<T, GK, K, V, MODE, HD>), grid, block, 0, stream, a)
    if (gkf32) {
        if (mode == PREP_FWD) HDLA_PREP_LAUNCH(true, PREP_FWD);
        else if (mode == PREP_BWD) HDLA_PREP_LAUNCH(true, PREP_BWD);
        else HDLA_PREP_LAUNCH(true, PREP_KEEP);
    } else {
        if (mode == PREP_FWD) HDLA_PREP_LAUNCH(kAlwaysF32, PREP_FWD);
        else if (mode == PREP_BWD) HDLA_PREP_LAUNCH(kAlwaysF32, PREP_BWD);
        else HDLA_PREP_LAUNCH(kAlwaysF32, PREP_KEEP);
    }
#undef HDLA_PREP_LAUNCH
    return hipGetLastError();
}

template <typename T, bool HD>
static hipError_t launch_prep_hd(const ChunkArgs<T>& a, int K, int V, int mode, hipStream_t stream) {
    if (K == 64 && V == 64) return launch_prep_kv<T, 64, 64, HD>(a, mode, stream);
    if (K == 128 && V == 128) return launch_prep_kv<T, 128, 128, HD>(a, mode, stream);
    if (K == 64 && V == 128) return launch_prep_kv<T, 64, 128, HD>(a, mode, stream);
    if (K == 128 && V == 64) return launch_prep_kv<T, 128, 64, HD>(a, mode, stream);
    return hipErrorInvalidValue;
}

template <typename T>
hipError_t launch_prep(const ChunkArgs<T>& a, int K, int V, int mode, hipStream_t stream) {
    return a.beta ? launch_prep_hd<T, true>(a, K, V, mode, stream) : launch_prep_hd<T, false>(a, K, V, mode, stream);
}
template hipError_t launch_prep<bf16>(const ChunkArgs<bf16>&, int, int, int, hipStream_t);
template hipError_t launch_prep<float>(const ChunkArgs<float>&, int, int, int, hipStream_t);

hipError_t launch_chunk_table(const int64_t* cu, int N, int T, int nch, int32_t* chunk_off, int32_t* chunk_seq, hipStream_t stream) {
    const int rankers = N <= ORDER_MAX_N ? (N + TABLE_THREADS - 1) / TABLE_THREADS : 0;
    hipLaunchKernelGGL(build_chunk_table_kernel, dim3(1 + rankers), dim3(TABLE_THREADS), 0, stream, cu, N, T, nch, chunk_off, chunk_seq);
    return hipGetLastError();
}

}  // namespace hdla
