// C ABI of libhdla_hip.so: argument checks, workspace layout and the launch sequences of the three entry points.
#include "../../include/hdla_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>

#include "fused_shapes.h"
#include "hdla_launch.h"
#include "hdla_ws.h"

using namespace hdla;

namespace {

constexpr int CHUNK = 16;

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// max_dim: 128 for the chunked entry points, 256 for the token-serial ones
int check_dims(const hdla_dims* d, int max_dim = 128) {
    if (!d) return HDLA_ERR_NULL;
    if (d->R != 2) return HDLA_ERR_RANK;
    if (d->B < 1 || d->T < 0 || d->H < 1 || d->N < 1) return HDLA_ERR_SHAPE;
    auto ok = [&](int x) { return x == 64 || x == 128 || (x == 256 && max_dim >= 256); };
    if (!ok(d->K) || !ok(d->V)) return HDLA_ERR_SHAPE;
    if (d->H > 65535) return HDLA_ERR_SHAPE;
    if (d->in_dtype != HDLA_BF16 && d->in_dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    if (d->gk_dtype != HDLA_BF16 && d->gk_dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    if (d->in_dtype == HDLA_FP32 && d->gk_dtype != HDLA_FP32) return HDLA_ERR_DTYPE;
    if (d->cu_seqlens) { if (d->B != 1) return HDLA_ERR_SEQ; }
    else if (d->N != d->B) return HDLA_ERR_SEQ;
    if (d->route < HDLA_ROUTE_AUTO || d->route > HDLA_ROUTE_FUSED || d->segments < 0) return HDLA_ERR_ROUTE;
    return HDLA_OK;
}

// ---- the fused route (fused_impl.cuh) ----------------------------------------------------------------------------
constexpr int FUSED_MAX_SEGMENTS = 64;       // the segments are chained serially by every workgroup that needs them: about a
                                             // microsecond a segment, against 2.5 for every chunk a segment is shorter
constexpr int FUSED_MIN_SEGMENT_CHUNKS = 8;  // a segment pays for its transition matrix: not worth it for a few chunks
constexpr int FUSED_TARGET_WORKGROUPS = 256; // one workgroup per compute unit

// the shapes the fused kernels are built for
bool fused_shape(const hdla_dims* d) { return d->in_dtype == HDLA_BF16 && d->K == 64 && d->V == 64; }
// whether the plain entry points take the fused route for these dimensions; HDLA_ROUTE_FUSED on another shape is an error
int pick_route(const hdla_dims* d, bool& fused) {
    fused = d->route != HDLA_ROUTE_CLASSIC && fused_shape(d);
    if (d->route == HDLA_ROUTE_FUSED && !fused) return HDLA_ERR_ROUTE;
    return HDLA_OK;
}
// time segments per sequence: as many as give every compute unit a workgroup, within the limits above
int fused_segments(const hdla_dims* d) {
    if (d->segments > 0) return d->segments < FUSED_MAX_SEGMENTS ? d->segments : FUSED_MAX_SEGMENTS;
    const long long lanes = (long long)d->N * d->H;
    const long long chunks_per_seq = ((d->T + CHUNK - 1) / CHUNK) / (d->cu_seqlens ? d->N : 1);
    int nseg = 1;
    while (nseg * 2 <= FUSED_MAX_SEGMENTS && lanes * nseg * 2 <= FUSED_TARGET_WORKGROUPS &&
           chunks_per_seq / (nseg * 2) >= FUSED_MIN_SEGMENT_CHUNKS) nseg *= 2;
    return nseg;
}

struct FusedLayout {
    size_t OL, GW, SLOC, MSEG, RSEG, SIN, ERR;                 // fused kernels' own
    size_t HC, DHC, DVN, TM, UT, W, STRONG;                    // what chunk_grad reads (backward pass)
    size_t CHUNK_OFF, CHUNK_SEQ;
    size_t total;
    int nch, nseg;
};
int make_fused_layout(const hdla_dims* d, int pass, FusedLayout& L) {
    const int rc = check_dims(d);
    if (rc) return rc;
    if (d->N > 65535) return HDLA_ERR_SHAPE;
    const int NT = (d->T + CHUNK - 1) / CHUNK;
    const long long nch64 = d->cu_seqlens ? (long long)NT + d->N : (long long)d->B * NT;
    if (nch64 * d->H > 0x7fff0000LL) return HDLA_ERR_SHAPE;
    L = FusedLayout{};
    L.nch = (int)nch64;
    L.nseg = fused_segments(d);
    const size_t es = 2, K = d->K, V = d->V;
    const size_t chw = (size_t)d->H * (size_t)L.nch, recs = (size_t)d->N * d->H * L.nseg;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up256(bytes); return o; };
    L.ERR = take(256);
    L.SLOC = take(recs * K * V * 4);
    L.MSEG = take(recs * K * K * 4);
    if (pass == HDLA_PASS_FWD) {
        L.OL = take(chw * 16 * V * 4);
        L.GW = take(chw * 16 * K * es);
    } else {
        L.RSEG = take(recs * K * V * 4);
        L.SIN = take(recs * K * V * 4);
        L.HC = take(chw * K * V * es);
        L.DHC = take(chw * K * V * es);
        L.DVN = take(chw * 2 * 16 * V * es);
        L.TM = take(chw * 1024 * es);
        L.UT = take(chw * 2 * V * 16 * es);
        L.W = take(chw * 2 * K * 16 * es);
        L.STRONG = take(chw * 4);
    }
    if (d->cu_seqlens) {
        L.CHUNK_OFF = take((size_t)(2 * d->N + 1) * 4);
        L.CHUNK_SEQ = take((size_t)(L.nch > 0 ? L.nch : 1) * 4);
    }
    L.total = off;
    return HDLA_OK;
}
size_t fused_boundary_bytes(const hdla_dims* d) {
    const int nseg = fused_segments(d);
    return nseg > 1 ? (size_t)d->N * d->H * nseg * d->K * d->V * 4 : 0;
}

// pass: HDLA_PASS_FWD, _BWD, _FWD_KEEP (a forward pass that leaves what the backward pass needs of it), _BWD_KEPT (the
// scratch of a backward pass that runs on such a workspace: only what its own scans write)
int make_layout(const hdla_dims* d, int pass, WsLayout& L, int& nch) {
    const int rc = check_dims(d);
    if (rc) return rc;
    if (d->N > 65535) return HDLA_ERR_SHAPE;
    const int NT = (d->T + CHUNK - 1) / CHUNK;
    const long long nch64 = d->cu_seqlens ? (long long)NT + d->N : (long long)d->B * NT;
    if (nch64 * d->H > 0x7fff0000LL) return HDLA_ERR_SHAPE;        // one workgroup per (chunk, head), one grid dimension (and room for the strided loops over them)
    nch = (int)nch64;
    const size_t es = d->in_dtype == HDLA_BF16 ? 2 : 4;
    const size_t chw = (size_t)d->H * (size_t)nch;
    const size_t K = d->K, V = d->V;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up256(bytes); return o; };
    L = WsLayout{};
    const bool prep_out = pass != HDLA_PASS_BWD_KEPT;             // what the prep kernel writes
    const bool with_o = pass == HDLA_PASS_FWD || pass == HDLA_PASS_FWD_KEEP;
    const bool bwd_parts = pass == HDLA_PASS_BWD || pass == HDLA_PASS_FWD_KEEP;
    const bool scan_out = pass == HDLA_PASS_BWD || pass == HDLA_PASS_BWD_KEPT;
    if (prep_out) {
        const BlkF bf = blk_fwd(d->K, (int)es, with_o);
        const size_t sa = take(chw * (size_t)bf.SIZE);
        L.SA_STRIDE = bf.SIZE;
        L.W = sa + bf.W; L.BGT = sa + bf.BGT; L.KGT = sa + bf.KGT; L.EGL = sa + bf.EGL;
        if (with_o) { L.QG = sa + bf.QG; L.AQB = sa + bf.AQB; L.AQK = sa + bf.AQK; }
        L.UT = take(chw * 2 * V * 16 * es);
        L.VTT = take(chw * V * 16 * es);
    }
    if (bwd_parts) {
        const BlkB bb = blk_bwd(d->K, (int)es);
        const size_t sb = take(chw * (size_t)bb.SIZE);
        L.SB_STRIDE = bb.SIZE;
        L.QGT = sb + bb.QGT; L.AQBT = sb + bb.AQBT;
        L.TM = take(chw * 1024 * es);
        L.STRONG = take(chw * 4);
    }
    if (scan_out) {
        L.HC = take(chw * K * V * es);
        L.DHC = take(chw * K * V * es);
        L.DVN = take(chw * 2 * 16 * V * es);
    }
    if (d->cu_seqlens && prep_out) {
        L.CHUNK_OFF = take((size_t)(2 * d->N + 1) * 4);          // chunk_off [N+1], then order [N]
        L.CHUNK_SEQ = take((size_t)(nch > 0 ? nch : 1) * 4);
    }
    L.total = off > 0 ? off : 256;
    return HDLA_OK;
}

// what the prep kernel writes (and the sequence tables) lives in `prep_ws`, laid out by LP; what the scans of the
// backward pass write lives in `scan_ws`, laid out by LS (the same buffer and layout unless the backward pass runs on a
// kept forward workspace)
template <typename T>
void bind_ws(ChunkArgs<T>& a, const hdla_dims* d, const WsLayout& LP, void* prep_ws, const WsLayout& LS, void* scan_ws, int nch) {
    char* base = static_cast<char*>(prep_ws);
    auto at = [&](size_t o) { return reinterpret_cast<T*>(base + o); };
    a.ws.W = at(LP.W); a.ws.UT = at(LP.UT); a.ws.KGT = at(LP.KGT); a.ws.BGT = at(LP.BGT); a.ws.VTT = at(LP.VTT);
    a.ws.QG = at(LP.QG); a.ws.AQK = at(LP.AQK); a.ws.AQB = at(LP.AQB);
    a.ws.AQBT = at(LP.AQBT); a.ws.QGT = at(LP.QGT);
    a.ws.EGL = reinterpret_cast<float*>(base + LP.EGL);
    a.ws.TM = at(LP.TM);
    a.ws.STRONG = reinterpret_cast<int32_t*>(base + LP.STRONG);
    a.ws.sa_stride = (int)LP.SA_STRIDE;
    char* sbase = static_cast<char*>(scan_ws);
    a.ws.HC = reinterpret_cast<T*>(sbase + LS.HC); a.ws.DHC = reinterpret_cast<T*>(sbase + LS.DHC);
    a.ws.DVN = reinterpret_cast<T*>(sbase + LS.DVN);
    a.st.cu = d->cu_seqlens;
    a.st.chunk_off = d->cu_seqlens ? reinterpret_cast<const int32_t*>(base + LP.CHUNK_OFF) : nullptr;
    a.st.chunk_seq = d->cu_seqlens ? reinterpret_cast<const int32_t*>(base + LP.CHUNK_SEQ) : nullptr;
    a.st.order = d->cu_seqlens ? a.st.chunk_off + d->N + 1 : nullptr;
    a.st.T = d->T;
    a.st.NT = (d->T + CHUNK - 1) / CHUNK;
    a.st.N = d->N;
    a.st.nch = nch;
}

inline bool bad_ws(const void* p, size_t have, size_t need) {
    return !p || (reinterpret_cast<uintptr_t>(p) & 255) || have < need;
}

// pass: HDLA_PASS_FWD / _BWD on `workspace`; HDLA_PASS_FWD_KEEP on `kept`; HDLA_PASS_BWD_KEPT on `kept` (read) and
// `workspace` (what the scans write)
template <typename T>
int run_chunk(const hdla_dims* d, int pass, const void* q, const void* k, const void* v, const void* a_,
              const void* b, const void* gk, const float* h0, void* o, float* ht, const void* d_o,
              const float* dht, void* dq, void* dk, void* dv, void* da, void* db, void* dgk, float* dh0,
              void* workspace, size_t workspace_bytes, hipStream_t stream, int stages = HDLA_STAGE_ALL,
              const void* beta = nullptr, void* dbeta = nullptr, void* kept = nullptr, size_t kept_bytes = 0) {
    WsLayout LP, LS;
    int nch = 0;
    const bool fwd = pass == HDLA_PASS_FWD || pass == HDLA_PASS_FWD_KEEP;
    const bool on_kept = pass == HDLA_PASS_FWD_KEEP || pass == HDLA_PASS_BWD_KEPT;
    int rc = make_layout(d, on_kept ? HDLA_PASS_FWD_KEEP : pass, LP, nch);
    if (rc) return rc;
    void* prep_ws = on_kept ? kept : workspace;
    if (bad_ws(prep_ws, on_kept ? kept_bytes : workspace_bytes, LP.total)) return HDLA_ERR_WORKSPACE;
    LS = LP;
    if (pass == HDLA_PASS_BWD_KEPT) {
        rc = make_layout(d, pass, LS, nch);
        if (rc) return rc;
        if (bad_ws(workspace, workspace_bytes, LS.total)) return HDLA_ERR_WORKSPACE;
    }
    ChunkArgs<T> a{};
    a.q = static_cast<const T*>(q); a.k = static_cast<const T*>(k); a.v = static_cast<const T*>(v);
    a.a = static_cast<const T*>(a_); a.b = static_cast<const T*>(b);
    a.gk = gk; a.gk_f32 = d->gk_dtype == HDLA_FP32;
    a.H = d->H; a.scale = d->scale;
    a.h0 = h0; a.ht = fwd ? ht : nullptr; a.o = static_cast<T*>(o);
    a.dout = static_cast<const T*>(d_o); a.dht = dht; a.dh0 = dh0;
    a.dq = static_cast<T*>(dq); a.dk = static_cast<T*>(dk); a.dv = static_cast<T*>(dv);
    a.da = static_cast<T*>(da); a.db = static_cast<T*>(db); a.dgk = dgk;
    a.beta = static_cast<const T*>(beta); a.dbeta = static_cast<T*>(dbeta);
    bind_ws(a, d, LP, prep_ws, LS, pass == HDLA_PASS_BWD_KEPT ? workspace : prep_ws, nch);
    hipError_t e;
    if (pass == HDLA_PASS_BWD_KEPT) stages &= ~HDLA_STAGE_PREP;    // the forward pass has run it
    if (d->cu_seqlens && (stages & HDLA_STAGE_PREP)) {
        char* base = static_cast<char*>(prep_ws);
        e = launch_chunk_table(d->cu_seqlens, d->N, d->T, nch, reinterpret_cast<int32_t*>(base + LP.CHUNK_OFF),
                               reinterpret_cast<int32_t*>(base + LP.CHUNK_SEQ), stream);
        if (e != hipSuccess) return (int)e;
    }
    if (nch > 0 && (stages & HDLA_STAGE_PREP)) {
        e = launch_prep<T>(a, d->K, d->V, pass == HDLA_PASS_FWD ? 0 : pass == HDLA_PASS_BWD ? 1 : 2, stream);
        if (e != hipSuccess) return (int)e;
    }
    // the two scans of the backward pass are independent of each other: one launch when both are asked for
    const bool pair = !fwd && (stages & HDLA_STAGE_SCAN_FWD) && (stages & HDLA_STAGE_SCAN_BWD);
    if (pair) {
        e = launch_scan_pair<T>(a, d->K, d->V, stream);
        if (e != hipSuccess) return (int)e;
    } else if (stages & HDLA_STAGE_SCAN_FWD) {
        e = launch_scan_fwd<T>(a, d->K, d->V, fwd, stream);
        if (e != hipSuccess) return (int)e;
    }
    if (!fwd) {
        if (!pair && (stages & HDLA_STAGE_SCAN_BWD)) {
            e = launch_scan_bwd<T>(a, d->K, d->V, stream);
            if (e != hipSuccess) return (int)e;
        }
        if (nch > 0 && (stages & HDLA_STAGE_CHUNK_GRAD)) {
            e = launch_chunk_grad<T>(a, d->K, d->V, stream);
            if (e != hipSuccess) return (int)e;
        }
    }
    return HDLA_OK;
}

// The fused route's launch sequences.  Forward: fused kernel (+ fixup kernel when there are several segments); it
// leaves the states entering the segments in `boundary` when given.  Backward: (without `boundary`: summary pass +
// chaining, to re-derive those states) checkpoint kernel, reverse kernel, chunk_grad.
int run_fused(const hdla_dims* d, bool fwd, const void* q, const void* k, const void* v, const void* a_, const void* b,
              const void* beta, const void* gk, const float* h0, void* o, float* ht, const void* d_o, const float* dht,
              void* dq, void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk, float* dh0, void* boundary,
              size_t boundary_bytes, void* workspace, size_t workspace_bytes, hipStream_t stream,
              int stages = HDLA_STAGE_ALL) {
    typedef bf16 T;
    FusedLayout L;
    const int rc = make_fused_layout(d, fwd ? HDLA_PASS_FWD : HDLA_PASS_BWD, L);
    if (rc) return rc;
    if (bad_ws(workspace, workspace_bytes, L.total)) return HDLA_ERR_WORKSPACE;
    if (boundary && (L.nseg > 1) && (boundary_bytes < fused_boundary_bytes(d) || (reinterpret_cast<uintptr_t>(boundary) & 15)))
        return HDLA_ERR_WORKSPACE;
    char* base = static_cast<char*>(workspace);
    FusedArgs<T> f{};
    ChunkArgs<T>& a = f.c;
    a.q = static_cast<const T*>(q); a.k = static_cast<const T*>(k); a.v = static_cast<const T*>(v);
    a.a = static_cast<const T*>(a_); a.b = static_cast<const T*>(b);
    a.gk = gk; a.gk_f32 = d->gk_dtype == HDLA_FP32;
    a.H = d->H; a.scale = d->scale;
    a.h0 = h0; a.ht = fwd ? ht : nullptr; a.o = static_cast<T*>(o);
    a.dout = static_cast<const T*>(d_o); a.dht = dht; a.dh0 = dh0;
    a.dq = static_cast<T*>(dq); a.dk = static_cast<T*>(dk); a.dv = static_cast<T*>(dv);
    a.da = static_cast<T*>(da); a.db = static_cast<T*>(db); a.dgk = dgk;
    a.beta = static_cast<const T*>(beta); a.dbeta = static_cast<T*>(dbeta);
    a.ws.HC = reinterpret_cast<T*>(base + L.HC); a.ws.DHC = reinterpret_cast<T*>(base + L.DHC);
    a.ws.DVN = reinterpret_cast<T*>(base + L.DVN); a.ws.TM = reinterpret_cast<T*>(base + L.TM);
    a.ws.UT = reinterpret_cast<T*>(base + L.UT); a.ws.W = reinterpret_cast<T*>(base + L.W);
    a.ws.STRONG = reinterpret_cast<int32_t*>(base + L.STRONG);
    a.ws.sa_stride = 2 * d->K * 16 * 2;                            // chunk_grad's view of w: [2][K/16] tiles per slot
    a.st.cu = d->cu_seqlens;
    a.st.chunk_off = d->cu_seqlens ? reinterpret_cast<const int32_t*>(base + L.CHUNK_OFF) : nullptr;
    a.st.chunk_seq = d->cu_seqlens ? reinterpret_cast<const int32_t*>(base + L.CHUNK_SEQ) : nullptr;
    a.st.order = d->cu_seqlens ? a.st.chunk_off + d->N + 1 : nullptr;
    a.st.T = d->T; a.st.NT = (d->T + CHUNK - 1) / CHUNK; a.st.N = d->N; a.st.nch = L.nch;
    f.nseg = L.nseg;
    f.sloc = reinterpret_cast<float*>(base + L.SLOC); f.mseg = reinterpret_cast<float*>(base + L.MSEG);
    f.rseg = reinterpret_cast<float*>(base + L.RSEG);
    f.err = reinterpret_cast<int*>(base + L.ERR);
    hipError_t e;
    if (d->cu_seqlens && (stages & HDLA_STAGE_PREP)) {
        e = launch_chunk_table(d->cu_seqlens, d->N, d->T, L.nch, reinterpret_cast<int32_t*>(base + L.CHUNK_OFF),
                               reinterpret_cast<int32_t*>(base + L.CHUNK_SEQ), stream);
        if (e != hipSuccess) return (int)e;
    }
    if (fwd) {
        f.ol = reinterpret_cast<float*>(base + L.OL); f.gw = reinterpret_cast<T*>(base + L.GW);
        f.sin_out = static_cast<float*>(boundary);
        if (stages & HDLA_STAGE_SCAN_FWD) {
            e = launch_fused<T>(f, d->K, d->V, FUSED_FWD, stream);
            if (e != hipSuccess) return (int)e;
        }
        if (L.nseg > 1 && (stages & HDLA_STAGE_CHAIN)) {
            e = launch_fixup<T>(f, d->K, d->V, stream);
            if (e != hipSuccess) return (int)e;
        }
        return HDLA_OK;
    }
    if (L.nseg > 1 && !boundary) {
        // inputs only: one pass for the segment records, chained into the states entering the segments (a caller that
        // runs the stages one by one may leave this one out once the workspace holds them)
        f.sin_out = reinterpret_cast<float*>(base + L.SIN);
        f.gw = nullptr;
        if (stages & HDLA_STAGE_CHAIN) {
            e = launch_fused<T>(f, d->K, d->V, FUSED_SUM, stream);
            if (e != hipSuccess) return (int)e;
            e = launch_fixup<T>(f, d->K, d->V, stream);
            if (e != hipSuccess) return (int)e;
        }
        f.sin = f.sin_out;
    } else {
        f.sin = static_cast<const float*>(boundary);
    }
    if (stages & HDLA_STAGE_SCAN_FWD) {
        e = launch_fused<T>(f, d->K, d->V, FUSED_CKPT, stream);
        if (e != hipSuccess) return (int)e;
    }
    if (stages & HDLA_STAGE_SCAN_BWD) {
        e = launch_fused<T>(f, d->K, d->V, FUSED_REV, stream);
        if (e != hipSuccess) return (int)e;
    }
    if (L.nch > 0 && (stages & HDLA_STAGE_CHUNK_GRAD)) {
        e = launch_chunk_grad<T>(a, d->K, d->V, stream);
        if (e != hipSuccess) return (int)e;
    }
    return HDLA_OK;
}

}  // namespace

// ---- scratch memory of the entry point that allocates nothing ------------------------------------------------
// One array per GPU, part of the loaded code object, held until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress; the address kernels can use is looked up once per device and kept here.
// (No `used` attribute on the array: with it the compiler keeps the symbol local to the code object, where the runtime's
// lookup by name fails; the host-side reference below is what keeps the array and makes its symbol visible.)
static __device__ __align__(256) unsigned char scratch[HDLA_STATIC_WORKSPACE_BYTES];
static constexpr int MAX_DEVICES = 64;
static std::atomic<void*> g_scratch_ptr[MAX_DEVICES];

// Device address of `scratch` on the current device (looked up on the first call per device); nullptr and *err set
// on failure.  Two threads racing on the first call both obtain the same address.
static void* static_scratch(int* err) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { *err = (int)e; return nullptr; }
    if (dev < 0 || dev >= MAX_DEVICES) { *err = HDLA_ERR_SHAPE; return nullptr; }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) { *err = e != hipSuccess ? (int)e : HDLA_ERR_WORKSPACE; return nullptr; }
    g_scratch_ptr[dev].store(p, std::memory_order_release);
    return p;
}

extern "C" {

int hdla_version(void) { return HDLA_VERSION; }

const char* hdla_strerror(int code) {
    switch (code) {
        case HDLA_OK: return "success";
        case HDLA_ERR_NULL: return "a required pointer is NULL";
        case HDLA_ERR_SHAPE: return "unsupported shape (need K,V in {64,128}, or 256 as well for the token-serial entry points; B,H,N >= 1, T >= 0, H,N <= 65535, chunks x heads < 2^31)";
        case HDLA_ERR_RANK: return "only rank R = 2 is supported";
        case HDLA_ERR_DTYPE: return "unsupported dtype (in_dtype bf16|fp32; gk fp32, or bf16 with bf16 inputs)";
        case HDLA_ERR_WORKSPACE: return "workspace is NULL, not 256-byte aligned, or smaller than hdla_workspace_bytes()";
        case HDLA_ERR_ALIGN: return "tensor pointers must be 16-byte aligned";
        case HDLA_ERR_SEQ: return "cu_seqlens needs B == 1; without it N must equal B";
        case HDLA_ERR_ROUTE: return "route must be HDLA_ROUTE_AUTO, _CLASSIC or _FUSED (the fused route: bf16 inputs, K = V = 64) and segments >= 0";
        case HDLA_ERR_STATIC_LIMIT: return "the call needs more scratch memory than the built-in HDLA_STATIC_WORKSPACE_BYTES; use hdla_chunk_fwd with a caller-owned workspace";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error code";
    }
}

size_t hdla_workspace_bytes(const hdla_dims* dims, int pass) {
    WsLayout L;
    int nch;
    if (pass < HDLA_PASS_FWD || pass > HDLA_PASS_BWD_KEPT) return 0;
    if (check_dims(dims)) return 0;
    bool fused;
    if (pick_route(dims, fused)) return 0;
    if (fused && (pass == HDLA_PASS_FWD || pass == HDLA_PASS_BWD)) {
        FusedLayout F;
        return make_fused_layout(dims, pass, F) ? 0 : F.total;
    }
    if (make_layout(dims, pass, L, nch)) return 0;
    return L.total;
}

size_t hdla_boundary_bytes(const hdla_dims* dims) {
    bool fused;
    if (check_dims(dims) || pick_route(dims, fused) || !fused) return 0;
    return fused_boundary_bytes(dims);
}

int hdla_workspace_layout(const hdla_dims* dims, int pass, hdla_ws_layout* out) {
    if (!out) return HDLA_ERR_NULL;
    if (pass < HDLA_PASS_FWD || pass > HDLA_PASS_BWD_KEPT) return HDLA_ERR_SHAPE;
    WsLayout L;
    int nch;
    int rc = check_dims(dims);
    if (rc) return rc;
    bool fused;
    rc = pick_route(dims, fused);
    if (rc) return rc;
    if (fused && (pass == HDLA_PASS_FWD || pass == HDLA_PASS_BWD)) {
        FusedLayout F;
        rc = make_fused_layout(dims, pass, F);
        if (rc) return rc;
        *out = hdla_ws_layout{};
        out->nch = F.nch;
        out->UT = F.UT; out->TM = F.TM; out->HC = F.HC; out->DHC = F.DHC; out->DVN = F.DVN; out->STRONG = F.STRONG;
        out->W = F.W; out->SA_STRIDE = pass == HDLA_PASS_BWD ? 2 * dims->K * 16 * 2 : 0;
        out->CHUNK_OFF = F.CHUNK_OFF; out->CHUNK_SEQ = F.CHUNK_SEQ;
        out->total = F.total;
        out->ERR = F.ERR;
        return HDLA_OK;
    }
    rc = make_layout(dims, pass, L, nch);
    if (rc) return rc;
    out->nch = nch;
    out->W = L.W; out->UT = L.UT; out->KGT = L.KGT; out->BGT = L.BGT; out->VTT = L.VTT; out->EGL = L.EGL;
    out->QG = L.QG; out->AQK = L.AQK; out->AQB = L.AQB;
    out->AQBT = L.AQBT; out->QGT = L.QGT; out->TM = L.TM;
    out->SA_STRIDE = L.SA_STRIDE; out->SB_STRIDE = L.SB_STRIDE;
    out->HC = L.HC; out->DHC = L.DHC; out->DVN = L.DVN; out->STRONG = L.STRONG;
    out->CHUNK_OFF = L.CHUNK_OFF; out->CHUNK_SEQ = L.CHUNK_SEQ;
    out->total = L.total;
    out->ERR = -1;
    return HDLA_OK;
}

// forward pass of either form (a, b given, or beta) on the route the dimensions select
static int chunk_fwd_any(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                         const void* beta, const void* gk, const float* h0, void* o, float* ht, void* boundary,
                         size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_dims(dims);
    if (rc) return rc;
    if (dims->T > 0 && (!q || !k || !v || !gk || !o || (!beta && (!a || !b)))) return HDLA_ERR_NULL;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(a) || !aligned16(b) || !aligned16(gk) ||
        !aligned16(o) || !aligned16(h0) || !aligned16(ht)) return HDLA_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (beta) { a = nullptr; b = nullptr; }
    bool fused;
    rc = pick_route(dims, fused);
    if (rc) return rc;
    if (fused)
        return run_fused(dims, true, q, k, v, a, b, beta, gk, h0, o, ht, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                         nullptr, nullptr, nullptr, nullptr, boundary, boundary_bytes, workspace, workspace_bytes, s);
    if (dims->in_dtype == HDLA_BF16)
        return run_chunk<bf16>(dims, 0, q, k, v, a, b, gk, h0, o, ht, nullptr, nullptr, nullptr, nullptr, nullptr,
                               nullptr, nullptr, nullptr, nullptr, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, nullptr);
    return run_chunk<float>(dims, 0, q, k, v, a, b, gk, h0, o, ht, nullptr, nullptr, nullptr, nullptr, nullptr,
                            nullptr, nullptr, nullptr, nullptr, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, nullptr);
}

static int chunk_bwd_any(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                         const void* beta, const void* gk, const float* h0, const void* d_o, const float* dht, void* dq,
                         void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk, float* dh0, const void* boundary,
                         size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_dims(dims);
    if (rc) return rc;
    if (dims->T > 0 && (!q || !k || !v || !gk || !d_o || !dq || !dk || !dv || !dgk)) return HDLA_ERR_NULL;
    if (dims->T > 0 && (beta ? !dbeta : (!a || !b || !da || !db))) return HDLA_ERR_NULL;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(a) || !aligned16(b) || !aligned16(gk) ||
        !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !aligned16(da) || !aligned16(db) ||
        !aligned16(dgk) || !aligned16(h0) || !aligned16(dht) || !aligned16(dh0)) return HDLA_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (beta) { a = nullptr; b = nullptr; da = nullptr; db = nullptr; }
    bool fused;
    rc = pick_route(dims, fused);
    if (rc) return rc;
    if (fused)
        return run_fused(dims, false, q, k, v, a, b, beta, gk, h0, nullptr, nullptr, d_o, dht, dq, dk, dv, da, db, dbeta, dgk,
                         dh0, const_cast<void*>(boundary), boundary_bytes, workspace, workspace_bytes, s);
    if (dims->in_dtype == HDLA_BF16)
        return run_chunk<bf16>(dims, 1, q, k, v, a, b, gk, h0, nullptr, nullptr, d_o, dht, dq, dk, dv, da, db, dgk,
                               dh0, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, dbeta);
    return run_chunk<float>(dims, 1, q, k, v, a, b, gk, h0, nullptr, nullptr, d_o, dht, dq, dk, dv, da, db, dgk,
                            dh0, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, dbeta);
}

int hdla_chunk_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                   const void* b, const void* gk, const float* h0, void* o, float* ht,
                   void* workspace, size_t workspace_bytes, void* stream) {
    if (dims && dims->T > 0 && (!a || !b)) return HDLA_ERR_NULL;
    return chunk_fwd_any(dims, q, k, v, a, b, nullptr, gk, h0, o, ht, nullptr, 0, workspace, workspace_bytes, stream);
}

int hdla_chunk_fwd_static(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                          const void* b, const void* gk, const float* h0, void* o, float* ht, void* stream) {
    const size_t need = hdla_workspace_bytes(dims, 0);
    if (need == 0) { const int rc = check_dims(dims); return rc ? rc : HDLA_ERR_SHAPE; }
    if (need > (size_t)HDLA_STATIC_WORKSPACE_BYTES) return HDLA_ERR_STATIC_LIMIT;
    int err = 0;
    void* ws = static_scratch(&err);
    if (!ws) return err;
    // every byte of the workspace that a kernel of the forward pass reads has been written by an earlier kernel of
    // the same call, so nothing has to be cleared between calls
    return hdla_chunk_fwd(dims, q, k, v, a, b, gk, h0, o, ht, ws, (size_t)HDLA_STATIC_WORKSPACE_BYTES, stream);
}

int hdla_chunk_bwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                   const void* b, const void* gk, const float* h0, const void* d_o, const float* dht,
                   void* dq, void* dk, void* dv, void* da, void* db, void* dgk, float* dh0,
                   void* workspace, size_t workspace_bytes, void* stream) {
    return chunk_bwd_any(dims, q, k, v, a, b, nullptr, gk, h0, d_o, dht, dq, dk, dv, da, db, nullptr, dgk, dh0, nullptr, 0,
                         workspace, workspace_bytes, stream);
}

int hdla_param_chunk_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                         const void* gk, const float* h0, void* o, float* ht,
                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!beta) return HDLA_ERR_NULL;
    return chunk_fwd_any(dims, q, k, v, nullptr, nullptr, beta, gk, h0, o, ht, nullptr, 0, workspace, workspace_bytes, stream);
}

int hdla_param_chunk_bwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                         const void* gk, const float* h0, const void* d_o, const float* dht,
                         void* dq, void* dk, void* dv, void* dbeta, void* dgk, float* dh0,
                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!beta) return HDLA_ERR_NULL;
    return chunk_bwd_any(dims, q, k, v, nullptr, nullptr, beta, gk, h0, d_o, dht, dq, dk, dv, nullptr, nullptr, dbeta, dgk,
                         dh0, nullptr, 0, workspace, workspace_bytes, stream);
}

int hdla_chunk_fwd_b(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                     const void* beta, const void* gk, const float* h0, void* o, float* ht, void* boundary,
                     size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream) {
    return chunk_fwd_any(dims, q, k, v, a, b, beta, gk, h0, o, ht, boundary, boundary_bytes, workspace, workspace_bytes, stream);
}

int hdla_chunk_bwd_b(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a, const void* b,
                     const void* beta, const void* gk, const float* h0, const void* d_o, const float* dht, void* dq,
                     void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk, float* dh0, const void* boundary,
                     size_t boundary_bytes, void* workspace, size_t workspace_bytes, void* stream) {
    return chunk_bwd_any(dims, q, k, v, a, b, beta, gk, h0, d_o, dht, dq, dk, dv, da, db, dbeta, dgk, dh0, boundary,
                         boundary_bytes, workspace, workspace_bytes, stream);
}

int hdla_chunk_fwd_keep(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                        const void* b, const void* beta, const void* gk, const float* h0, void* o, float* ht,
                        void* kept, size_t kept_bytes, void* stream) {
    const int rc = check_dims(dims);
    if (rc) return rc;
    if (dims->T > 0 && (!q || !k || !v || !gk || !o || (!beta && (!a || !b)))) return HDLA_ERR_NULL;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(a) || !aligned16(b) || !aligned16(gk) ||
        !aligned16(o) || !aligned16(h0) || !aligned16(ht)) return HDLA_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (beta) { a = nullptr; b = nullptr; }
    if (dims->in_dtype == HDLA_BF16)
        return run_chunk<bf16>(dims, HDLA_PASS_FWD_KEEP, q, k, v, a, b, gk, h0, o, ht, nullptr, nullptr, nullptr, nullptr,
                               nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, s, HDLA_STAGE_ALL, beta, nullptr,
                               kept, kept_bytes);
    return run_chunk<float>(dims, HDLA_PASS_FWD_KEEP, q, k, v, a, b, gk, h0, o, ht, nullptr, nullptr, nullptr, nullptr,
                            nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, s, HDLA_STAGE_ALL, beta, nullptr,
                            kept, kept_bytes);
}

int hdla_chunk_bwd_kept(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                        const void* b, const void* beta, const void* gk, const float* h0, const void* d_o,
                        const float* dht, void* dq, void* dk, void* dv, void* da, void* db, void* dbeta, void* dgk,
                        float* dh0, void* kept, size_t kept_bytes, void* workspace, size_t workspace_bytes,
                        void* stream) {
    const int rc = check_dims(dims);
    if (rc) return rc;
    if (dims->T > 0 && (!q || !k || !v || !gk || !d_o || !dq || !dk || !dv || !dgk)) return HDLA_ERR_NULL;
    if (dims->T > 0 && (beta ? !dbeta : (!a || !b || !da || !db))) return HDLA_ERR_NULL;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(a) || !aligned16(b) || !aligned16(gk) ||
        !aligned16(d_o) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv) || !aligned16(da) || !aligned16(db) ||
        !aligned16(dgk) || !aligned16(h0) || !aligned16(dht) || !aligned16(dh0)) return HDLA_ERR_ALIGN;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (beta) { a = nullptr; b = nullptr; da = nullptr; db = nullptr; }
    if (dims->in_dtype == HDLA_BF16)
        return run_chunk<bf16>(dims, HDLA_PASS_BWD_KEPT, q, k, v, a, b, gk, h0, nullptr, nullptr, d_o, dht, dq, dk, dv, da,
                               db, dgk, dh0, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, dbeta, kept, kept_bytes);
    return run_chunk<float>(dims, HDLA_PASS_BWD_KEPT, q, k, v, a, b, gk, h0, nullptr, nullptr, d_o, dht, dq, dk, dv, da,
                            db, dgk, dh0, workspace, workspace_bytes, s, HDLA_STAGE_ALL, beta, dbeta, kept, kept_bytes);
}

int hdla_chunk_stages(const hdla_dims* dims, int pass, int stages, const void* q, const void* k, const void* v,
                      const void* a, const void* b, const void* gk, const float* h0, void* o, float* ht,
                      const void* d_o, const float* dht, void* dq, void* dk, void* dv, void* da, void* db, void* dgk,
                      float* dh0, void* workspace, size_t workspace_bytes, void* stream) {
    const int rc = check_dims(dims);
    if (rc) return rc;
    if (pass != 0 && pass != 1) return HDLA_ERR_SHAPE;
    if (!q || !k || !v || !a || !b || !gk) return HDLA_ERR_NULL;
    if (pass == 0 ? !o : (!d_o || !dq || !dk || !dv || !da || !db || !dgk)) return HDLA_ERR_NULL;
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool fused;
    const int rr = pick_route(dims, fused);
    if (rr) return rr;
    if (fused)
        return run_fused(dims, pass == 0, q, k, v, a, b, nullptr, gk, h0, o, ht, d_o, dht, dq, dk, dv, da, db, nullptr, dgk, dh0,
                         nullptr, 0, workspace, workspace_bytes, s, stages);
    if (dims->in_dtype == HDLA_BF16)
        return run_chunk<bf16>(dims, pass, q, k, v, a, b, gk, h0, o, ht, d_o, dht, dq, dk, dv, da, db, dgk, dh0,
                               workspace, workspace_bytes, s, stages);
    return run_chunk<float>(dims, pass, q, k, v, a, b, gk, h0, o, ht, d_o, dht, dq, dk, dv, da, db, dgk, dh0,
                            workspace, workspace_bytes, s, stages);
}

static int run_recurrent(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                         const void* b, const void* beta, const void* gk, int reverse, const float* h0, void* o,
                         float* ht, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (dims->in_dtype == HDLA_BF16) {
        RecurrentArgs<bf16> r{};
        r.q = static_cast<const bf16*>(q); r.k = static_cast<const bf16*>(k); r.v = static_cast<const bf16*>(v);
        r.a = static_cast<const bf16*>(a); r.b = static_cast<const bf16*>(b);
        r.beta = static_cast<const bf16*>(beta);
        r.gk = gk; r.gk_f32 = dims->gk_dtype == HDLA_FP32;
        r.H = dims->H; r.T_ = dims->T; r.N = dims->N; r.scale = dims->scale; r.reverse = reverse;
        r.cu = dims->cu_seqlens; r.h0 = h0; r.ht = ht; r.o = static_cast<bf16*>(o);
        e = launch_recurrent<bf16>(r, dims->K, dims->V, s);
    } else {
        RecurrentArgs<float> r{};
        r.q = static_cast<const float*>(q); r.k = static_cast<const float*>(k); r.v = static_cast<const float*>(v);
        r.a = static_cast<const float*>(a); r.b = static_cast<const float*>(b);
        r.beta = static_cast<const float*>(beta);
        r.gk = gk; r.gk_f32 = 1;
        r.H = dims->H; r.T_ = dims->T; r.N = dims->N; r.scale = dims->scale; r.reverse = reverse;
        r.cu = dims->cu_seqlens; r.h0 = h0; r.ht = ht; r.o = static_cast<float*>(o);
        e = launch_recurrent<float>(r, dims->K, dims->V, s);
    }
    return e == hipSuccess ? HDLA_OK : (int)e;
}

int hdla_recurrent_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* a,
                       const void* b, const void* gk, int reverse, const float* h0, void* o, float* ht,
                       void* stream) {
    const int rc = check_dims(dims, 256);
    if (rc) return rc;
    if (dims->T > 0 && (!q || !k || !v || !a || !b || !gk || !o)) return HDLA_ERR_NULL;
    if (!aligned16(h0) || !aligned16(ht)) return HDLA_ERR_ALIGN;
    return run_recurrent(dims, q, k, v, a, b, nullptr, gk, reverse, h0, o, ht, stream);
}

int hdla_param_recurrent_fwd(const hdla_dims* dims, const void* q, const void* k, const void* v, const void* beta,
                             const void* gk, int reverse, const float* h0, void* o, float* ht, void* stream) {
    const int rc = check_dims(dims, 256);
    if (rc) return rc;
    if (!beta) return HDLA_ERR_NULL;
    if (dims->T > 0 && (!q || !k || !v || !gk || !o)) return HDLA_ERR_NULL;
    if (!aligned16(h0) || !aligned16(ht)) return HDLA_ERR_ALIGN;
    return run_recurrent(dims, q, k, v, nullptr, nullptr, beta, gk, reverse, h0, o, ht, stream);
}

}  // extern "C"
