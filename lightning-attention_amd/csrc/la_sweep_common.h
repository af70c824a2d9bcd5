// Definitions shared by the sweep kernels (bf16 / fp16 MFMA paths).
#pragma once
#include "la_common.h"
#include "lightning_attn_hip.h"

namespace la {

// How the caller wants a call mapped onto launches (all zero: the library's own choices).
typedef la_launch_opts Opts;

// Where the (batch, head, token) rows of a tensor start, in elements; the feature dim is contiguous.
// A plain (b, h, n, d) tensor has {h*n*d, n*d, d}; a (b, n, h, d) projection output viewed as
// (b, h, n, d) has {n*h*d, d, h*d}.
struct Layout {
    int64_t bs, hs, ts;  // batch, head, token stride
};

struct SweepArgs {
    const void* x;  // (b, h, n, dk)
    const void* y;  // (b, h, n, dk)
    const void* z;  // (b, h, n, dv)
    void* out;      // (b, h, n, dv)
    Layout lx, ly, lz, lo;
    const float* s; // h decay rates or nullptr
    int64_t n;
    int dk, dv, h, bh, nslice;
    int zw;              // columns of z / out per slice: 64, or - 128-column workgroups - a multiple of 32 up to 128
    int nchunk;          // sequence chunks per (batch, head, slice); 1 = one workgroup walks the whole sequence
    int chunk_start[9];  // first 64-token block (in walk order) of each chunk; chunk_start[nchunk] = number of blocks
};

// Bounds-checked buffer over the rows of one (batch, head) sequence of a tensor with `cols` features.
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t seq_rsrc(const void* p, const Layout& l, int unit, int h, int64_t n, int cols) {
    const T* base = static_cast<const T*>(p) + (int64_t)(unit / h) * l.bs + (int64_t)(unit % h) * l.hs;
    return make_rsrc(base, (unsigned)(((n - 1) * l.ts + cols) * (int64_t)sizeof(T)));
}

template <typename T>
struct Mma;
template <>
struct Mma<__bf16> {
    typedef bf16x8 V8;
    typedef bf16x4 V4;
    static __device__ __forceinline__ f32x4 mma(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ __bf16 cvt(float f) { return (__bf16)f; }
};
template <>
struct Mma<_Float16> {
    typedef f16x8 V8;
    typedef f16x4 V4;
    static __device__ __forceinline__ f32x4 mma(V8 a, V8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    // fp16 saturates instead of overflowing to inf when a state entry is large
    static __device__ __forceinline__ _Float16 cvt(float f) {
        return (_Float16)__builtin_fminf(__builtin_fmaxf(f, -65504.f), 65504.f);
    }
};

// LDS transpose read: the 16 lanes of a group each point at 4 consecutive
// 16-bit elements; lane i of the group receives element (i % 4) of the lanes
// 4e + i/4, e = 0..3.  With lane L pointing at row L/4, columns 4(L%4).. of a
// row-major tile, lane i ends up with column i of rows 0..3.
template <typename V4>
__device__ __forceinline__ V4 lds_tr4(const void* p) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
    return __builtin_bit_cast(V4, v);
}
template <typename V8, typename V4>
__device__ __forceinline__ V8 cat(V4 a, V4 b) {
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// The 10 non-masked 16x16 tiles of the 64x64 score block, dealt to the four score
// waves: slot 0 is tile (jt0, itA), slots 1,2 are (jt1, itB), (jt2, itB); -1 = none.
// Written for the forward direction (jt <= it); the reverse direction mirrors
// both indices (3 - jt, 3 - it).
struct TileDeal {
    int itA, jt0, itB, jt1, jt2;
};
__device__ __constant__ const TileDeal kDeal[4] = {
    {3, 0, 3, 1, 2},
    {3, 3, 2, 0, 1},
    {2, 2, 1, 0, 1},
    {0, 0, -1, -1, -1},
};

// Operands of one sweep: x, y (b, h, n, dk), z, out (b, h, n, dv), each with its own layout.
struct SweepIO {
    const void *x, *y, *z;
    void* out;
    Layout lx, ly, lz, lo;
};

// One launch of the pipelined kernel can carry two sweeps of the same shape, direction and layout
// kind (dK and dV of the backward pass when d == e).  Their workgroups for one (batch, head) sit
// next to each other on one XCD and walk the sequence in step, so the tensors the two sweeps have in
// common (dO and Q) come from memory once and from that XCD's L2 the second time.
struct SweepPair {
    SweepArgs a[2];
    int nprod;  // 1 or 2 sweeps; a[1] is unused when 1
    int wide;   // pipelined kernel only: a workgroup covers 128 instead of 64 columns of z / out
    // How a chunk's workgroup gets the state its chunk starts from:
    //   kWarmUp   it walks the blocks before its chunk with the state update only (no workspace);
    //   kCollect  first of three launches: every workgroup walks its own chunk, state update only, starting
    //             from zero, and leaves the state it ends with in `state` (the last chunk has nothing to leave);
    //   kApply    third launch: it starts from `state`, which the scan kernel run in between has turned
    //             into the state at the start of each chunk.
    //   kResume   a single launch: it starts from `state`, which an earlier sweep over the same y and z in
    //             swapped roles has left behind (`save` below).
    // In the three latter modes the chunks are chunk_len blocks long (a[0].chunk_start is not used).  kCollect /
    // kApply: `state` holds, per (unit, sweep, slice), nchunk - 1 slots of the state waves' accumulators.
    // kResume: per unit nchunk - 1 plain row-major matrices of dv x dk floats, matrix c - 1 being the
    // transpose of the state chunk c starts from (pipelined kernel, 128-column workgroups, one sweep).
    int mode;
    int chunk_len;
    float* state;
    // Forward walk in one piece (pipelined kernel, 64-column workgroups): after every save_len blocks but the
    // last the state is also written to `save`, per unit (number of such boundaries) row-major dk x dv float
    // matrices.  The sweep (x', y' = z, z' = y) then has exactly the transposed state at those boundaries
    // and can start chunks there (kResume): the dQ sweep of the backward pass after the forward pass.
    // nullptr / 0: nothing is saved.
    float* save = nullptr;
    int save_len = 0;
    // x, y and z are pre-activations: the kernel applies SiLU to them as it loads them (forward sweeps of
    // the pipelined kernel at feature dims up to 128)
    int silu = 0;
};

// One launch can also carry sweeps of both directions: the whole backward pass when d == e, dQ walking
// forward, dK and dV backward.  That pays when the three sweeps together leave CUs idle (few
// sequences): they run side by side instead of one after the other.  Warm-up chunking only; both
// parts use the same kernel instantiation (64 columns per workgroup).
struct SweepBoth {
    SweepPair fwd, rev;
    unsigned nfwd;  // workgroups of the forward part (a multiple of 8); the reverse part follows
};
int sweep_pipe_both(const SweepBoth& b, int dtype, hipStream_t st);  // la_sweep_pipe.hip
// Workgroups of one part of such a launch (units are dealt to the 8 XCDs, so their number is rounded up to 8).
inline unsigned part_grid(const SweepPair& p) {
    return (unsigned)((p.a[0].bh + 7) / 8 * 8 * p.a[0].nslice * p.a[0].nchunk * p.nprod);
}

// Count (up to 8) and first blocks, chunk_start[0 .. 8], of the warm-up chunks for a launch that would have
// `wgs` workgroups with one chunk each, on a walk of nblk blocks; `forced` > 0 overrides the count.
// Defined in la_sweep.hip.
void plan_warm_up_chunks(int64_t wgs, int64_t nblk, int forced, int* nchunk, int* chunk_start);

// Raises a kernel's dynamic LDS limit above the 64 KB default, once per kernel and device (the call is
// not free and the limit stays).  `done` is the instantiation's own flag array, one entry per device.
template <typename K>
inline int allow_lds(K kern, size_t lds, unsigned char (&done)[kMaxDevices]) {
    if (lds <= 64 * 1024) return 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const bool cached = dev >= 0 && dev < kMaxDevices;
    if (cached && __atomic_load_n(&done[dev], __ATOMIC_ACQUIRE)) return 0;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    if (cached) __atomic_store_n(&done[dev], (unsigned char)1, __ATOMIC_RELEASE);
    return 0;
}

// Where a forward pass leaves states for the backward pass's dQ sweep (la_sweep.hip): chunks of that sweep,
// their length in blocks (= blocks between two saved states), bytes of float matrices; nchunk == 1: nowhere.
struct SavedPlan {
    int nchunk, chunk_len;
    size_t bytes;
    int fwd_width, dq_width;  // columns per workgroup (width code of SweepPair::wide) of the pass that saves / resumes
};

// Launches the single-barrier pipelined kernel (feature dim up to 256); defined in la_sweep_pipe.hip.
// n, dk, dv, h, bh, nslice and the chunking must agree between the two sweeps of a pair.
enum { kWarmUp = 0, kCollect = 1, kApply = 2, kResume = 3 };
int sweep_pipe(const SweepPair& p, int dtype, bool reverse, hipStream_t st);
// One-time work per device, done ahead of the first launches: the dynamic LDS limits of every instantiation
// of the pipelined kernels (la_sweep_pipe.hip) and of the float32 kernels (la_sweep_f32.hip), and the
// device's compute-unit count (la_sweep.hip).
int prepare_pipe();
int prepare_f32();
int prepare_plans();
// Floats of one state slot: the feature dim as the kernel pads it (64, 128, 192 or 256) times the 64 or 128
// columns of a workgroup.  Must agree with the kernels' own SF; the 128-column form pads feature dims up
// to 64 to 128.
inline size_t pipe_state_floats(int dk, int wide) {
    const int dkp = dk > 192 ? 256 : dk > 128 ? 192 : (dk <= 64 && !wide ? 64 : 128);
    return (size_t)dkp * (wide == 2 ? 192 : wide ? 128 : 64);
}
// Between a kCollect and a kApply launch: scans the chunks' end states in place (la_sweep_pipe.hip).
int launch_state_scan(const SweepPair& p, hipStream_t st);
}  // namespace la
