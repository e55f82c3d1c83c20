// chunk_grad kernel: everything of the backward pass that is local to one 16-token chunk.
//
// One workgroup of four wavefronts per (chunk, head) fuses what the reference runs as five launches: the dA part of
// HRDPLR/bwd_triton.py:30-105, the dv kernel :239-290, the dqg/dkg/dbg/dw/dgk_last kernel :309-487, the WY
// backward :503-612, the score backward :627-883 and the log-decay gradient :899-948.  Its inputs are the
// original tensors, do, and per chunk the state entering it (h), the gradient of the state leaving it (dh) and
// the gradient of v_new, left in the workspace by the two scans, and (I - A_ab)^-1 and u from the prep kernel (w as
// well with the HDLA parameterisation; otherwise it is rebuilt here).  Nothing but the seven gradients is written back.
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
    // all tiles of w (2 ranks), rebuilt by the waves from (I - A_ab)^-1 and a instead of read from the workspace: behind
    // the sums above, in what is otherwise free until the staged rows are written
    static constexpr int WALL_B = 2 * (K / 16) * TILE * ES;
    // per wave and token: three partial sums over channels of the backward of the HDLA parameterisation
    static constexpr int RED = KG + KG_B, RED_B = NW * 3 * CH * 4;
    static constexpr int R1 = RED + RED_B, WALL = R1 + PART_B, R1_B = PART_B + WALL_B > OUT_B ? PART_B + WALL_B : OUT_B;
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

// The common kernel: one workgroup per (chunk, head); pairs flagged for the strong-decay route are left alone.
template <typename T, bool GKF32, int K, int V, bool HD>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(cg_waves<T, GKF32, K, V, HD>(false), cg_waves<T, GKF32, K, V, HD>(true)))) void chunk_grad_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[CgLds<T, K, V>::BYTES];
    // Which of the two indices runs fastest over the workgroups decides which rows of the [token][head][channel]
    // tensors the workgroups resident at one time touch.  Measured: with rows of 4 KiB and more, neighbouring
    // workgroups should be the heads of one chunk (together they read whole rows; chunk-fastest, all of them would
    // touch the same few hundred bytes of every row, a fraction of the HBM channels); with shorter rows the chunks
    // of one head, whose workspace records are contiguous.
    const bool head_fastest = (uint32_t)(p.H * K) * sizeof(T) >= 4096;
    const int cid = head_fastest ? blockIdx.x / p.H : blockIdx.x % p.st.nch;
    const int h = head_fastest ? blockIdx.x % p.H : blockIdx.x / p.st.nch;
#define CG_STRONG 0
#include "chunk_grad_body.inc"
#undef CG_STRONG
}

template <typename T, bool GKF32, int K, int V, bool HD>
__device__ __forceinline__ void chunk_grad_strong_pair(const ChunkArgs<T>& p, int cid, int h, char* smem) {
#define CG_STRONG 1
#include "chunk_grad_body.inc"
#undef CG_STRONG
}

// The kernel for the flagged pairs.  They are rare (a channel must lose more than e^-70 within eight tokens), so this
// is a small fixed grid whose workgroups each look through their share of the flags (one read per thread and round)
// and work off what they find one pair after the other, at one wave per SIMD with all the registers the three passes
// want; when nothing is flagged, which is the rule, the launch costs its start-up and one round of flag reads.  The
// common kernel sits at the register limit of three workgroups per compute unit and pays nothing for this one.
constexpr int CG_STRONG_GRID = 256;
template <typename T, bool GKF32, int K, int V, bool HD>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(1, 1))) void chunk_grad_strong_kernel(ChunkArgs<T> p) {
    __shared__ __attribute__((aligned(16))) char smem[CgLds<T, K, V>::BYTES];
    __shared__ unsigned long long sMask[NW];
    const int total = p.H * p.st.nch, nth = 64 * NW;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int base = blockIdx.x; base < total; base += (int)gridDim.x * nth) {      // uniform over the workgroup
        const int mine = base + (int)threadIdx.x * (int)gridDim.x;
        const unsigned long long m = __ballot(mine < total && p.ws.STRONG[mine] != 0);
        if (lane_id() == 0) sMask[w] = m;
        __syncthreads();
        for (int ww = 0; ww < NW; ++ww) {
            unsigned long long todo = sMask[ww];                                   // uniform: the same word for all
            while (todo) {
                const int t = 64 * ww + __builtin_ctzll(todo);
                todo &= todo - 1;
                const int chw = base + t * (int)gridDim.x;
                chunk_grad_strong_pair<T, GKF32, K, V, HD>(p, chw % p.st.nch, chw / p.st.nch, smem);
                __syncthreads();                                                   // the next pair reuses the staging areas
            }
        }
        __syncthreads();
    }
}

template <typename T, int K, int V, bool HD>
static hipError_t launch_chunk_grad_kv(const ChunkArgs<T>& a, hipStream_t stream) {
    dim3 grid(a.st.nch * a.H), block(64 * NW);
    constexpr bool kAlwaysF32 = sizeof(T) == 4;
    const int total = a.st.nch * a.H;
    dim3 sgrid(total < CG_STRONG_GRID ? total : CG_STRONG_GRID);
    if (kAlwaysF32 || a.gk_f32) {
        hipLaunchKernelGGL((chunk_grad_kernel<T, true, K, V, HD>), grid, block, 0, stream, a);
        hipLaunchKernelGGL((chunk_grad_strong_kernel<T, true, K, V, HD>), sgrid, block, 0, stream, a);
    } else {
        hipLaunchKernelGGL((chunk_grad_kernel<T, kAlwaysF32, K, V, HD>), grid, block, 0, stream, a);
        hipLaunchKernelGGL((chunk_grad_strong_kernel<T, kAlwaysF32, K, V, HD>), sgrid, block, 0, stream, a);
    }
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
