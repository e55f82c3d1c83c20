// Workspace layout and kernel argument blocks shared by the kernels and the C-ABI host code.
//
// Every per-chunk buffer is laid out [head][chunk slot][per-chunk elements]: the chunks of one (sequence, head)
// are contiguous, which is the order the two state scans walk them in.  Buffers marked "tiles" hold 16x16 tiles
// in fragment order (lane-major, 256 elements per tile) so that the consumer reads back exactly the registers
// the producer held; buffers marked "rows" are plain row-major.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace hdla {

struct bf16 { uint16_t x; };  // storage type tag for bf16 tensors (raw bits)

// Tokens live on one flattened axis of B*T rows.  Without cu_seqlens sequence n covers rows [n*T, (n+1)*T) and
// has NT = ceil(T/16) chunks; with cu_seqlens (device int64[N+1], batch 1) sequence n covers [cu[n], cu[n+1])
// and its chunks are numbered from chunk_off[n] (device int32[N+1], built by build_chunk_table_kernel, which leaves
// the int32[N] `order` right behind it).
struct SeqTab {
    const int64_t* cu;        // nullable
    const int32_t* chunk_off; // valid when cu != nullptr
    const int32_t* chunk_seq; // valid when cu != nullptr: sequence of each chunk
    const int32_t* order;     // valid when cu != nullptr: int32[N], the sequences from the one with the most chunks down
    int T, NT, N;
    int nch;                  // chunk slots the workspace is laid out for (an upper bound with cu_seqlens)
};

// Operands of the state scans that all value-column blocks of a (chunk, head) share are kept in ONE contiguous
// block per (chunk, head), so that a workgroup can copy a block into LDS with a few whole-kilobyte loads.
// Byte offsets inside a block, by head size K, element size es and pass:
//   forward-scan block:  W [2][K/16] | BGT [2][K/16] | KGT [K/16] | EGL fp32[K] (one 1-KiB piece) | (QG [K/16] | AQB [2])
//                        with AQK [1] in the second half of the EGL piece (2-byte elements) or in a piece of its own
//   reverse-scan block:  QGT [K/16] | AQBT [2]       (the reverse scan also reads W, BGT and EGL of the forward-scan
//                        block and turns the tiles of W and BGT itself)
// (tiles of 256 elements in fragment order, consecutive tile pairs interleaved; the part in parentheses and AQK only
// where the scan also produces the output.  The block without that part is a prefix of the block with it, so the
// kernels of the backward pass can work on blocks a forward pass left behind: only the distance between blocks differs.)
struct BlkF { int W, BGT, KGT, QG, AQB, AQK, EGL, SIZE; };
struct BlkB { int QGT, AQBT, SIZE; };
constexpr BlkF blk_fwd(int K, int es, bool with_o) {
    const int tb = 256 * es, KT = K / 16;
    BlkF b{};
    b.W = 0; b.BGT = 2 * KT * tb; b.KGT = 4 * KT * tb; b.EGL = 5 * KT * tb;
    const int egl_end = b.EGL + 1024;                    // 4 K <= 512 bytes of decay factors, rounded to a piece
    if (with_o) {
        b.AQK = es == 2 ? b.EGL + 512 : egl_end;
        b.QG = es == 2 ? egl_end : egl_end + tb;
        b.AQB = b.QG + KT * tb;
        b.SIZE = (b.AQB + 2 * tb + 1023) & ~1023;
    } else {
        b.QG = 0; b.AQB = 0; b.AQK = 0;
        b.SIZE = egl_end;
    }
    return b;
}
constexpr BlkB blk_bwd(int K, int es) {
    const int tb = 256 * es, KT = K / 16;
    BlkB b{};
    b.QGT = 0; b.AQBT = KT * tb;
    b.SIZE = ((KT + 2) * tb + 1023) & ~1023;
    return b;
}

// LDS slot of the reverse scan, assembled from 1-KiB pieces of both blocks of a (chunk, head): W and BGT (the first
// NIF pieces of the forward-scan block), the piece holding EGL, then the reverse-scan block.
struct SlotB { int W, BGT, EGL, QGT, AQBT, SIZE, NIF, EGL_SRC; };
constexpr SlotB slot_bwd(int K, int es) {
    const int tb = 256 * es, KT = K / 16;
    SlotB s{};
    s.W = 0; s.BGT = 2 * KT * tb; s.NIF = 4 * KT * tb / 1024;
    s.EGL = s.NIF * 1024; s.EGL_SRC = blk_fwd(K, es, false).EGL;      // EGL is 1 KiB aligned in the forward block
    s.QGT = s.EGL + 1024; s.AQBT = s.QGT + KT * tb;
    s.SIZE = s.QGT + blk_bwd(K, es).SIZE;
    return s;
}

// Byte offsets into the caller's workspace; 0-sized entries are unused in the given pass.  The entries of the
// two scan blocks (W .. EGL and QGT, AQBT) are the offsets of that part for (chunk, head) slot 0; consecutive
// slots are SA_STRIDE / SB_STRIDE bytes apart.
struct WsLayout {
    // written by prep, read by the scans
    size_t W;      // tiles  [2][K/16]   F(w_s)        rows token, inner channel
    size_t UT;     // tiles  [2][V/16]   F(u_s^T)      rows value, inner token
    size_t KGT;    // tiles  [K/16]      F(kg^T)       rows channel, inner token
    size_t BGT;    // tiles  [2][K/16]   F(bg_s^T)     rows channel, inner token
    size_t VTT;    // tiles  [V/16]      F(v^T)        rows value, inner token
    size_t EGL;    // fp32   [K]         exp(g_last)
    // forward pass only
    size_t QG;     // tiles  [K/16]      F(qg)         rows token, inner channel
    size_t AQK;    // tiles  [1]         F(A_qk)       rows i, inner j
    size_t AQB;    // tiles  [2]         F(A_qb^s)     rows i, inner j
    // backward pass only
    size_t AQBT;   // tiles  [2]         F(A_qb^s^T)   rows j, inner i
    size_t QGT;    // tiles  [K/16]      F(qg^T)       rows channel, inner token
    size_t SA_STRIDE, SB_STRIDE;   // bytes between consecutive (chunk, head) slots of the two scan blocks
    size_t TM;     // tiles  [2][2]      F((Tm^{s r})^T), Tm = (I - A_ab)^-1 in 16x16 blocks: rows j, inner i
    size_t HC;     // tiles  [K/32][V/16] pairs  F(S^T), state entering the chunk: rows value, inner channel
    size_t DHC;    // tiles  [K/32][V/16] pairs  the same for the gradient of the state leaving the chunk
    size_t DVN;    // tiles  [V/16] pairs        F(dv_new_s^T), the two ranks paired: rows value, inner token
    size_t STRONG; // int32  [1]         nonzero: a channel of this (chunk, head) decays beyond SAFE_RANGE within the chunk
    // chunk table (only with cu_seqlens)
    size_t CHUNK_OFF;  // int32 [N+1]
    size_t CHUNK_SEQ;  // int32 [nch]
    size_t total;
};

template <typename T>
struct Ws {
    T *W, *UT, *KGT, *BGT, *VTT, *QG, *AQK, *AQB, *AQBT, *QGT, *HC, *DHC, *DVN;
    float *EGL;
    T* TM;
    int32_t* STRONG;
    int sa_stride;            // bytes between the forward-scan blocks of consecutive (chunk, head) slots
};

template <typename T>
struct ChunkArgs {            // inputs of the chunked operator + workspace
    const T *q, *k, *v, *a, *b;
    // HDLA parameterisation (hdla_custom.py:19-43): when beta is given, a and b are not read but formed in the
    // kernels from (beta, k, gk), and the backward pass returns dbeta (and folds da, db into dk, dgk) instead of da, db
    const T* beta;            // nullable [B,T,H]
    T* dbeta;
    const void* gk;
    int gk_f32;
    int H;
    float scale;
    SeqTab st;
    Ws<T> ws;
    // forward scan
    const float* h0;          // nullable [N][H][K][V]
    float* ht;                // nullable
    T* o;                     // forward pass output
    // backward
    const T* dout;            // do [B,T,H,V]
    const float* dht;         // nullable
    float* dh0;               // nullable
    T *dq, *dk, *dv, *da, *db;
    void* dgk;
};

template <typename T>
struct RecurrentArgs {
    const T *q, *k, *v, *a, *b;
    const T* beta;            // non-null: a, b formed per token from (beta, k, gk); a and b are not read
    const void* gk;
    int gk_f32;
    int H, T_, N;
    float scale;
    int reverse;
    const int64_t* cu;        // nullable, device
    const float* h0;          // nullable
    float* ht;                // nullable
    T* o;
};

}  // namespace hdla
