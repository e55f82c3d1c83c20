// Shared device-side building blocks of the HDLA rank-2 DPLR delta-rule kernels for gfx950 (CDNA4, wave64).
//
// Everything in the chunked path is phrased as products of 16x16 tiles held in MFMA register fragments.
// A "row fragment" F(X) of a 16 x 16 tile X is 4 values per lane: lane (g, c) = (lane / 16, lane % 16)
// holds X[c][4g .. 4g+3], i.e. row c, four consecutive entries of the inner (contracted) dimension.
//
//     mm(F(P), F(Q), acc)   accumulates   Z = P * Q^T   as a row fragment:  lane (g,c) reg i  +=  Z[c][4g+i]
//
// so the rows of the first argument become the rows of the result and the rows of the second argument become
// the inner index of the result.  The result of one product is therefore directly the operand of the next one
// (after conversion to the operand type), which is what lets the inter-chunk state scan run entirely in
// registers.  The two instantiations are bf16 operands (v_mfma_f32_16x16x16_bf16) and fp32 operands
// (four v_mfma_f32_16x16x4_f32 steps with the inner index permuted to match); both accumulate in fp32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hdla_ws.h"

namespace hdla {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int CH = 16;       // tokens per chunk
constexpr int MID = 7;       // token whose cumulative log-decay centres the factorised scores
constexpr int RANK = 2;      // rank of the a/b update
constexpr int TILE = 256;    // elements of one 16x16 tile (64 lanes x 4)

template <typename T> struct Frag;
template <> struct Frag<bf16> { s16x4 v; };
template <> struct Frag<float> { f32x4 v; };

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// ---- conversions -------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf2f(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ uint16_t f2bf(float f) {
    // round to nearest even; inputs here are finite by construction
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(uint16_t, h);
}

template <typename T> __device__ __forceinline__ Frag<T> to_frag(f32x4 a);
template <> __device__ __forceinline__ Frag<bf16> to_frag<bf16>(f32x4 a) {
    // two v_cvt_pk_bf16_f32 (round to nearest even), results already packed in operand order
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    const f32x2 lo = {a[0], a[1]}, hi = {a[2], a[3]};
    u32x2 w;
    w[0] = __builtin_bit_cast(unsigned, __builtin_convertvector(lo, bf16x2));
    w[1] = __builtin_bit_cast(unsigned, __builtin_convertvector(hi, bf16x2));
    Frag<bf16> r;
    r.v = __builtin_bit_cast(s16x4, w);
    return r;
}
template <> __device__ __forceinline__ Frag<float> to_frag<float>(f32x4 a) { Frag<float> r; r.v = a; return r; }

__device__ __forceinline__ f32x4 to_f32(Frag<bf16> a) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 w = __builtin_bit_cast(u32x2, a.v);
    f32x4 r;
    r[0] = __uint_as_float(w[0] << 16); r[1] = __uint_as_float(w[0] & 0xffff0000u);
    r[2] = __uint_as_float(w[1] << 16); r[3] = __uint_as_float(w[1] & 0xffff0000u);
    return r;
}
__device__ __forceinline__ f32x4 to_f32(Frag<float> a) { return a.v; }

// Tells the optimiser that x may have changed (it has not, and no instruction is emitted): what is computed from x
// after this point stays after it, in particular inside a loop in which x does not change, instead of being hoisted
// out of the loop and kept in registers across it.
__device__ __forceinline__ void pin(Frag<bf16>& x) { asm volatile("" : "+v"(x.v)); }
__device__ __forceinline__ void pin(Frag<float>&) {}     // fp32 operands are used as they are: nothing to hoist

__device__ __forceinline__ f32x4 zero4() { f32x4 z = {0.f, 0.f, 0.f, 0.f}; return z; }

// ---- the tile product --------------------------------------------------------------------------------------
// acc[lane(g,c)][i] += sum_k P[c][k] * Q[4g+i][k]     (frows = F(P), finner = F(Q))
__device__ __forceinline__ f32x4 mm(Frag<bf16> frows, Frag<bf16> finner, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(finner.v, frows.v, acc, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mm(Frag<float> frows, Frag<float> finner, f32x4 acc) {
#pragma unroll
    for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(finner.v[s], frows.v[s], acc, 0, 0, 0);
    return acc;
}

// (The 16x16x32 bf16 MFMA of gfx950 would do two of these products in the time of one.  It is not used: built with
// it, the state scans gave wrong results that depended on the register allocation, while a kernel of nothing but
// such products was exact; the cause was not established, and no kernel here is bound by its matrix products.)

// Split operands for the score products of the bf16 path: x = hi + lo with both halves bf16, and
// P Q^T ~ Ph Qh^T + Ph Ql^T + Pl Qh^T, which removes the rounding of the decayed operands (the largest single
// contribution to the forward error) at the price of two more MFMAs per product.  fp32 operands need no split.
template <typename T> struct Split;
template <> struct Split<bf16> { Frag<bf16> hi, lo; };
template <> struct Split<float> { Frag<float> hi; };
__device__ __forceinline__ void split(f32x4 x, Split<bf16>& s) {
    s.hi = to_frag<bf16>(x);
    s.lo = to_frag<bf16>(x - to_f32(s.hi));
}
__device__ __forceinline__ void split(f32x4 x, Split<float>& s) { s.hi.v = x; }
__device__ __forceinline__ f32x4 mm3(const Split<bf16>& p, const Split<bf16>& q, f32x4 acc) {
    acc = mm(p.lo, q.hi, acc);
    acc = mm(p.hi, q.lo, acc);
    return mm(p.hi, q.hi, acc);
}
__device__ __forceinline__ f32x4 mm3(const Split<float>& p, const Split<float>& q, f32x4 acc) { return mm(p.hi, q.hi, acc); }

// F(I16): used to transpose a tile with one product, F(X^T) = mm(F(I), F(X)).
template <typename T> __device__ __forceinline__ Frag<T> ident_frag() {
    const int l = lane_id(), g = l >> 4, c = l & 15;
    f32x4 e;
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = (c == 4 * g + i) ? 1.f : 0.f;
    return to_frag<T>(e);
}
template <typename T> __device__ __forceinline__ Frag<T> transpose(Frag<T> x, Frag<T> ident) {
    return to_frag<T>(mm(ident, x, zero4()));
}

// Address = uniform base (it stays in scalar registers) + a 32-bit byte offset per lane.  This is the form the
// global memory instructions take directly: one address register per lane instead of two, no 64-bit vector adds.
template <typename T> __device__ __forceinline__ T* at(T* ubase, uint32_t byte_off) {
    return reinterpret_cast<T*>(reinterpret_cast<char*>(ubase) + byte_off);
}
template <typename T> __device__ __forceinline__ const T* at(const T* ubase, uint32_t byte_off) {
    return reinterpret_cast<const T*>(reinterpret_cast<const char*>(ubase) + byte_off);
}

// ---- fragment loads / stores -------------------------------------------------------------------------------
// four consecutive elements at p (8-byte aligned for bf16, 16-byte aligned for fp32)
__device__ __forceinline__ Frag<bf16> ld_frag(const bf16* p) { Frag<bf16> r; r.v = *reinterpret_cast<const s16x4*>(p); return r; }
__device__ __forceinline__ Frag<float> ld_frag(const float* p) { Frag<float> r; r.v = *reinterpret_cast<const f32x4*>(p); return r; }
__device__ __forceinline__ void st_frag(bf16* p, Frag<bf16> f) { *reinterpret_cast<s16x4*>(p) = f.v; }
__device__ __forceinline__ void st_frag(float* p, Frag<float> f) { *reinterpret_cast<f32x4*>(p) = f.v; }
template <typename T> __device__ __forceinline__ Frag<T> zero_frag() { return to_frag<T>(zero4()); }

// Masked load without a branch: p must be a readable address on every lane (callers clamp the row index);
// lanes with ok == false get zeros by a select after the load.  A branch around the load would stop the
// compiler from batching the loads of an unrolled loop, so every load would pay its own memory latency.
template <typename T> __device__ __forceinline__ Frag<T> ld_frag_sel(const T* p, bool ok) {
    Frag<T> f = ld_frag(p);
    Frag<T> z = zero_frag<T>();
    Frag<T> r;
    r.v = ok ? f.v : z.v;
    return r;
}

// one element stores (used for the strided, 4-rows-per-lane writes of row-major checkpoints)
__device__ __forceinline__ void st_elem(bf16* p, float x) { p->x = f2bf(x); }
__device__ __forceinline__ void st_elem(float* p, float x) { *p = x; }
__device__ __forceinline__ float ld_elem(const bf16* p) { return bf2f(p->x); }
__device__ __forceinline__ float ld_elem(const float* p) { return *p; }

// whole tile in fragment order: lane l owns elements [4l, 4l+4) of a 256-element block
template <typename T> __device__ __forceinline__ Frag<T> ld_tile(const T* tile) { return ld_frag(tile + 4 * lane_id()); }
template <typename T> __device__ __forceinline__ void st_tile(T* tile, Frag<T> f) { st_frag(tile + 4 * lane_id(), f); }

// Two tiles that one consumer lane always needs together are stored interleaved as a pair (1024 bytes for bf16):
// element 8*lane + 4*which + i, so that both fragments arrive with one 16-byte load per lane.  The scans are
// limited by the number of memory instructions a wave may have in flight, not by bytes.
typedef short s16x8 __attribute__((ext_vector_type(8)));
constexpr int PAIR = 2 * TILE;
__device__ __forceinline__ void ld_pair(const bf16* pair, Frag<bf16>& f0, Frag<bf16>& f1) {
    const s16x8 x = *reinterpret_cast<const s16x8*>(pair + 8 * lane_id());
    f0.v = __builtin_shufflevector(x, x, 0, 1, 2, 3);
    f1.v = __builtin_shufflevector(x, x, 4, 5, 6, 7);
}
__device__ __forceinline__ void ld_pair(const float* pair, Frag<float>& f0, Frag<float>& f1) {
    f0.v = *reinterpret_cast<const f32x4*>(pair + 8 * lane_id());
    f1.v = *reinterpret_cast<const f32x4*>(pair + 8 * lane_id() + 4);
}
template <typename T> __device__ __forceinline__ Frag<T> ld_pair_one(const T* pair, int which) {
    return ld_frag(pair + 8 * lane_id() + 4 * which);
}
template <typename T> __device__ __forceinline__ void st_pair(T* pair, int which, Frag<T> f) {
    st_frag(pair + 8 * lane_id() + 4 * which, f);
}
// both tiles of a pair at once: whole 16-byte pieces, so no cache line is ever written in two halves
__device__ __forceinline__ void st_pair2(bf16* pair, Frag<bf16> f0, Frag<bf16> f1) {
    const s16x8 x = __builtin_shufflevector(f0.v, f1.v, 0, 1, 2, 3, 4, 5, 6, 7);
    *reinterpret_cast<s16x8*>(pair + 8 * lane_id()) = x;
}
__device__ __forceinline__ void st_pair2(float* pair, Frag<float> f0, Frag<float> f1) {
    *reinterpret_cast<f32x4*>(pair + 8 * lane_id()) = f0.v;
    *reinterpret_cast<f32x4*>(pair + 8 * lane_id() + 4) = f1.v;
}

// gk may be stored as bf16 or fp32 independently of the other inputs (compile-time switch GKF32);
// same contract as ld_frag_sel: the address is readable on every lane, masked lanes read zero.
template <bool GKF32> __device__ __forceinline__ f32x4 ld_gk4(const void* base, int64_t elem_off, bool ok) {
    f32x4 x;
    if (GKF32) x = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(base) + elem_off);
    else x = to_f32(ld_frag(reinterpret_cast<const bf16*>(base) + elem_off));
    return ok ? x : zero4();
}
template <bool GKF32> __device__ __forceinline__ void st_gk4(void* base, int64_t elem_off, f32x4 x) {
    if (GKF32) *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(base) + elem_off) = x;
    else st_frag(reinterpret_cast<bf16*>(base) + elem_off, to_frag<bf16>(x));
}

// ---- exp: fast hardware exp2 for the bf16 path, full-accuracy expf for the fp32 path -----------------------
template <typename T> __device__ __forceinline__ float exp_t(float x);
template <> __device__ __forceinline__ float exp_t<bf16>(float x) { return __expf(x); }
template <> __device__ __forceinline__ float exp_t<float>(float x) { return expf(x); }
template <typename T> __device__ __forceinline__ f32x4 exp4(f32x4 x) {
    f32x4 r; r[0] = exp_t<T>(x[0]); r[1] = exp_t<T>(x[1]); r[2] = exp_t<T>(x[2]); r[3] = exp_t<T>(x[3]); return r;
}

// ---- sequence / chunk addressing ---------------------------------------------------------------------------
struct ChunkPos {
    int64_t tok0;  // first token row of the chunk on the flattened axis
    int len;       // valid tokens in the chunk (1..16)
    int n;         // sequence
};

// A value that is the same on every lane of the wave, moved to scalar registers.  What is read from a table arrives in
// vector registers even when the index is uniform; addresses formed from it would then be 64-bit vector arithmetic
// for every access, where a scalar base and a 32-bit lane offset do.
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ int64_t uniform(int64_t x) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)x >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Token rows [bos, eos) of packed sequence n, forced into 0 <= bos <= eos <= total: the table comes from the caller
// and is not validated on the device, and no value in it may take an access outside the tensors.
__device__ __forceinline__ void packed_bounds(const int64_t* cu, int n, int64_t total, int64_t& bos, int64_t& eos) {
    bos = min(max(cu[n], (int64_t)0), total);
    eos = min(max(cu[n + 1], bos), total);
}

// (cid: the same on every lane)
__device__ __forceinline__ bool locate_chunk(const SeqTab& st, int cid, ChunkPos& cp) {
    if (st.cu == nullptr) {
        if (cid >= st.N * st.NT) return false;
        cp.n = cid / st.NT;
        const int ic = cid - cp.n * st.NT;
        cp.tok0 = (int64_t)cp.n * st.T + (int64_t)ic * CH;
        cp.len = min(CH, st.T - ic * CH);
        return true;
    }
    if (cid >= uniform(st.chunk_off[st.N])) return false;
    cp.n = uniform(st.chunk_seq[cid]);
    const int ic = cid - uniform(st.chunk_off[cp.n]);
    int64_t bos, eos;
    packed_bounds(st.cu, cp.n, st.T, bos, eos);
    cp.tok0 = uniform(bos) + (int64_t)ic * CH;
    cp.len = (int)min((int64_t)CH, uniform(eos) - cp.tok0);
    return cp.len > 0;
}

// chunk range [c0, c1) of sequence n (n: the same on every lane)
__device__ __forceinline__ void seq_chunks(const SeqTab& st, int n, int& c0, int& c1) {
    if (st.cu == nullptr) { c0 = n * st.NT; c1 = c0 + st.NT; }
    else { c0 = uniform(st.chunk_off[n]); c1 = uniform(st.chunk_off[n + 1]); }
}

// token rows [bos, eos) of sequence n on the flattened axis (n: the same on every lane)
__device__ __forceinline__ void seq_bounds(const SeqTab& st, int n, int64_t& bos, int64_t& eos) {
    if (st.cu == nullptr) { bos = (int64_t)n * st.T; eos = bos + st.T; }
    else {
        packed_bounds(st.cu, n, st.T, bos, eos);
        bos = uniform(bos);
        eos = uniform(eos);
    }
}

// ---- per-chunk decay quantities in fragment layout ---------------------------------------------------------
// lane (g,c) holds token c of the chunk and channels 16*kt + 4g + i.  The 16 lanes of a group are one DPP "row",
// so prefix sums, suffix sums and sums over the tokens of a chunk are row_shr / row_shl / mirror additions on
// the vector ALU (out-of-row lanes read 0), with no LDS round trips.
template <int CTRL> __device__ __forceinline__ float dpp0(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ f32x4 dpp0(f32x4 x) {
    f32x4 r; r[0] = dpp0<CTRL>(x[0]); r[1] = dpp0<CTRL>(x[1]); r[2] = dpp0<CTRL>(x[2]); r[3] = dpp0<CTRL>(x[3]); return r;
}
__device__ __forceinline__ f32x4 scan16_incl(f32x4 x) {     // inclusive prefix sum over the 16 lanes of a group
    x += dpp0<0x111>(x);    // row_shr:1
    x += dpp0<0x112>(x);    // row_shr:2
    x += dpp0<0x114>(x);    // row_shr:4
    x += dpp0<0x118>(x);    // row_shr:8
    return x;
}
__device__ __forceinline__ f32x4 rscan16_incl(f32x4 x) {    // inclusive suffix sum over the 16 lanes of a group
    x += dpp0<0x101>(x);    // row_shl:1
    x += dpp0<0x102>(x);
    x += dpp0<0x104>(x);
    x += dpp0<0x108>(x);
    return x;
}
__device__ __forceinline__ f32x4 sum16(f32x4 x) {           // sum over the 16 lanes of a group, on all of them
    x += dpp0<0xB1>(x);     // quad_perm:[1,0,3,2]
    x += dpp0<0x4E>(x);     // quad_perm:[2,3,0,1]
    x += dpp0<0x141>(x);    // row_half_mirror
    x += dpp0<0x140>(x);    // row_mirror
    return x;
}
__device__ __forceinline__ f32x4 bcast16(f32x4 x, int src) {  // value of lane `src` of the own 16-lane group
    f32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = __shfl(x[i], src, 16);
    return r;
}
// the same with a compile-time source lane: one DPP move per register (row_newbcast), no LDS round trip
template <int SRC> __device__ __forceinline__ f32x4 bcast16(f32x4 x) {
    f32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        r[i] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x[i]), 0x150 + SRC, 0xf, 0xf, false));
    return r;
}
// value held by the lane 32 positions away (v_permlane32_swap exchanges the two halves of the wave)
__device__ __forceinline__ float xor32(float x) {
    const int xi = __float_as_int(x);
    auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    return __int_as_float(lane_id() < 32 ? r[1] : r[0]);
}

// value held by the lane 16 positions away within each half of the wave (v_permlane16_swap exchanges odd and even
// rows of 16 lanes between two registers)
__device__ __forceinline__ float xor16(float x) {
    const int xi = __float_as_int(x);
    auto r = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);     // r[0] rows: x0 x0 x2 x2, r[1]: x1 x1 x3 x3
    return __int_as_float((lane_id() & 16) ? r[0] : r[1]);
}
// sum over the four lanes c, c+16, c+32, c+48, on all of them
__device__ __forceinline__ float sum_groups(float x) {
    x += xor16(x);
    x += xor32(x);
    return x;
}


// ---- decay factors of the factorised score products --------------------------------------------------------------
// A score sums q_i[ch] k_j[ch] exp(gi_i[ch] - gi_j[ch]) over channels (j <= i; likewise with a, ge on the row side and b
// on the inner side).  To be a matrix product the decay must factorise: exp(gi_i - m) exp(m - gi_j) with a centre m per
// channel.  One centre (gi of token MID) serves the whole 16 x 16 tile as long as no exponent gi_i - m, ge_i - m exceeds
// SAFE_RANGE in magnitude: the factors then stay within e^+-70, inside the range of the element types with room for
// the operands themselves.  Beyond that (a channel that loses more than e^-70 over eight tokens) exp(gi_i - m) would
// overflow for pairs on one side of the centre, so the tile is assembled from three products whose exponents are all
// <= 0 or bounded:
//   pass 0: rows 8..15 x inner 0..7, centre token 7: gi_i - m <= 0 and m - gi_j <= 0, exact;
//   pass 1: rows 0..7 x inner 0..7, centre token 3;      pass 2: rows 8..15 x inner 8..15, centre token 11:
//           inside a half the per-token log-decay is clamped at -PASS_CLAMP first, so no exponent exceeds 4 tokens x
//           PASS_CLAMP = 80.  A pair (i, j) whose span holds a clamped token has weight < e^-20 = 2e-9 either way, and
//           every other pair is exact, so each weight is within 2e-9 (absolute) of its true value.
// Tokens outside a pass's rows / inner range get the factor 0, and what the passes leave above the diagonal is removed
// by the causal masks as before.
constexpr float SAFE_RANGE = 70.f;
constexpr float PASS_CLAMP = 20.f;

template <int N> __device__ __forceinline__ bool strong_decay(const f32x4 (&gi)[N], const f32x4 (&ge)[N]) {
    float big = 0.f;
#pragma unroll
    for (int kt = 0; kt < N; ++kt) {
        const f32x4 m = bcast16<MID>(gi[kt]);
#pragma unroll
        for (int i = 0; i < 4; ++i) big = fmaxf(big, fmaxf(fabsf(gi[kt][i] - m[i]), fabsf(ge[kt][i] - m[i])));
    }
    return __any(big > SAFE_RANGE) != 0;                 // the same answer on every lane of the wave
}

struct DecayPass {
    static constexpr int COUNT = 3;
    int centre;          // token whose cumulative decay centres the pass
    bool rows, cols;     // does this lane's token take part on the row side (q, a) / on the inner side (k, b)
    bool clamp;
    __device__ __forceinline__ DecayPass(int ps, int c) {
        centre = ps == 0 ? MID : ps == 1 ? MID / 2 : MID + (CH - MID) / 2;
        rows = ps == 1 ? c <= MID : c > MID;
        cols = ps == 2 ? c > MID : c <= MID;
        clamp = ps != 0;
    }
    // gi, ge: inclusive / exclusive cumulative log-decay of the lane's token (four channels)
    template <typename T> __device__ __forceinline__ void factors(f32x4 gi, f32x4 ge, f32x4& eq, f32x4& ek, f32x4& ea) const {
        if (clamp) {                                      // uniform over the wave
            f32x4 g = gi - ge;
#pragma unroll
            for (int i = 0; i < 4; ++i) g[i] = fmaxf(g[i], -PASS_CLAMP);
            gi = scan16_incl(g);
            ge = gi - g;
        }
        const f32x4 m = bcast16(gi, centre);
        const f32x4 z = zero4();
        f32x4 dq = gi - m, dk = m - gi, da = ge - m;
#pragma unroll
        for (int i = 0; i < 4; ++i) { dq[i] = fminf(dq[i], 80.f); dk[i] = fminf(dk[i], 80.f); da[i] = fminf(da[i], 80.f); }
        eq = rows ? exp4<T>(dq) : z;
        ek = cols ? exp4<T>(dk) : z;
        ea = rows ? exp4<T>(da) : z;
    }
};

}  // namespace hdla
