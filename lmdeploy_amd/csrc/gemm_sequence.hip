// A sequence of decode (up to 16 tokens) W4A16 GEMMs in ONE persistent launch.
//
// One grid of one workgroup per CU walks the whole list of GEMMs (a layer: qkv, o, gate/up, down; or
// several layers).  Each workgroup computes its strip of column tiles of every GEMM with the code of
// the one-GEMM strip kernel (strip_body.h), so results are bit-identical to it.
//
// A GEMM that reads what an earlier one wrote starts behind a device-wide barrier: outputs are written
// at agent scope (write-through; the eight XCDs' L2 caches are not coherent for ordinary stores),
// every wave drains its stores, the workgroup arrives on a two-level counter tree (32 leaf counters,
// then one root: 256 arrivals on a single address take 3.7 us, through the tree 1.7 us), the last
// arrival publishes the barrier's number in a flag word and everybody else polls that flag;
// afterwards activations and residuals are read at agent scope.  Before a workgroup arrives, every
// wave requests the weight tiles and (scale, zero) words of the first two groups it will work on in the
// next GEMM - weights depend on nothing - so HBM keeps streaming while the barrier is crossed.
//
// What it buys (measured, Llama-2-7B layer at 8 tokens): nothing.  The barrier with its store drain
// and the agent-scope read of the new activations costs what a kernel launch inside a HIP graph
// costs, about 3 us per GEMM.  The entry point therefore launches one kernel per GEMM unless the
// caller asks for the persistent launch.
//
// The waits are bounded: a workgroup that does not see the flag within the time limit sets an
// error word, stops waiting at this and every later barrier, and finishes normally (its results
// are then undefined).  That can only happen when the grid is not resident all at once, e.g.
// because another kernel holds CUs for longer than the limit.  Counters are reset by the last
// workgroup to leave, so the next launch finds them zero.
#include "strip_body.h"

#include <algorithm>
#include <cstdlib>

namespace w4a16 {

namespace {

using namespace strip;

constexpr int kLeaves = 32;

struct SeqArgs {
    SeqGemm   g[kSeqMax];
    int       count;
    int       T;
    int*      sync;        // kSyncInts ints, zero between launches
    long long spin_ticks;  // time limit of one barrier wait, in ticks of the device's wall clock
};

// sync area, in 64-int (256-byte) lines: [root][32 leaves][flag][done][error]
__device__ __forceinline__ int* sync_root(int* s) { return s; }
__device__ __forceinline__ int* sync_leaf(int* s, int i) { return s + 64 * (1 + i); }
__device__ __forceinline__ int* sync_flag(int* s) { return s + 64 * (kLeaves + 1); }
__device__ __forceinline__ int* sync_done(int* s) { return s + 64 * (kLeaves + 2); }
__device__ __forceinline__ int* sync_error(int* s) { return s + 64 * (kLeaves + 3); }
static_assert(64 * (kLeaves + 4) <= kSyncInts, "sync area too small");

// Device-wide barrier number `no` (0, 1, ...) of this launch; called by one thread per workgroup.
__device__ __forceinline__ void grid_arrive_and_wait(int* s, int no, long long spin_ticks)
{
    const int nwg     = gridDim.x;
    const int leaf    = blockIdx.x % kLeaves;
    const int leaves  = min(kLeaves, nwg);
    const int members = nwg / kLeaves + (leaf < nwg % kLeaves ? 1 : 0);
    const int old = __hip_atomic_fetch_add(sync_leaf(s, leaf), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == (no + 1) * members - 1) {
        const int o2 = __hip_atomic_fetch_add(sync_root(s), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (o2 == (no + 1) * leaves - 1) {
            __hip_atomic_store(sync_flag(s), no + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
    if (__hip_atomic_load(sync_error(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return;  // already given up
    const long long t0 = wall_clock64();
    for (;;) {
        if (__hip_atomic_load(sync_flag(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > no) return;
        if (wall_clock64() - t0 >= spin_ticks) break;
        __builtin_amdgcn_s_sleep(1);
    }
    __hip_atomic_store(sync_error(s), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Execution barrier of the workgroup with LDS traffic settled, but without waiting for global loads
// (__syncthreads would wait for every load in flight, and the first weight tiles of a GEMM are meant to
// stay in flight while the workgroup crosses the device-wide barrier).
__device__ __forceinline__ void workgroup_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The strip of workgroup `bx` in a matrix of NT column tiles dealt to `strips` workgroups per pass.
struct Strip {
    int col0, width;
};
__device__ __forceinline__ Strip strip_of(int NT, int strips, int passes, int pass, int bx)
{
    const int total = strips * passes;
    const int base = NT / total, rem = NT % total;
    const int idx = pass * strips + bx;
    return Strip{idx * base + min(idx, rem), base + (idx < rem ? 1 : 0)};
}

template<int TP>
__global__ void __launch_bounds__(64 * kWaves) sequence_kernel(const SeqArgs a)
{
    // activation patches [8][TP][16] / partial sums [8][R][64], as in the strip kernel
    extern __shared__ __attribute__((aligned(16))) u32x4_t smem[];
    const int tid    = threadIdx.x;
    const int bx     = blockIdx.x;
    const int strips = gridDim.x;

    int barrier_no = 0;
    for (int i = 0; i < a.count; ++i) {
        const SeqGemm& g      = a.g[i];
        const int      NT     = g.N / kTileN;
        const int      passes = (NT + strips * kMaxR - 1) / (strips * kMaxR);
        for (int pass = 0; pass < passes; ++pass) {
            // this wave's output stores of the previous unit are complete (written through to memory)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const Strip st = strip_of(NT, strips, passes, pass, bx);
            StripParams p{g.C, g.A, g.X, g.Q, g.R, g.N, a.T, g.K, 0, 0, g.epilogue, 1};
            // called by every wave once its first weight loads are on their way
            auto ready = [&]() {
                workgroup_barrier();  // every wave has drained its stores and is done with the sums in LDS
                if (pass == 0 && i > 0 && (g.flags & 1)) {
                    if (tid == 0) grid_arrive_and_wait(a.sync, barrier_no, a.spin_ticks);
                    ++barrier_no;
                    workgroup_barrier();
                }
            };
            switch (st.width) {
                case 1: strip_body<1, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 2: strip_body<2, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 3: strip_body<3, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 4: strip_body<4, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 5: strip_body<5, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 6: strip_body<6, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 7: strip_body<7, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                case 8: strip_body<8, TP, kEpiRuntime, true>(p, st.col0, smem, ready); break;
                default: ready(); break;  // fewer column tiles than workgroups: nothing to compute in this one
            }
        }
    }
    // the last workgroup to leave finds every other one past its last wait: it puts the counters back to zero
    if (tid == 0 && barrier_no > 0) {
        const int old = __hip_atomic_fetch_add(sync_done(a.sync), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (int)gridDim.x - 1) {
            for (int l = 0; l < kLeaves; ++l)
                __hip_atomic_store(sync_leaf(a.sync, l), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_root(a.sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_flag(a.sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_done(a.sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Measurement aid: `iters` device-wide barriers and nothing else.  tree = 0 lets every workgroup arrive on
// the root counter (what the two-level tree is there to avoid).
__global__ void __launch_bounds__(64 * kWaves) barrier_probe_kernel(int* sync, int iters, int tree, long long spin_ticks)
{
    for (int no = 0; no < iters; ++no) {
        if (threadIdx.x == 0) {
            if (tree) {
                grid_arrive_and_wait(sync, no, spin_ticks);
            }
            else {
                const int old = __hip_atomic_fetch_add(sync_root(sync), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (old == (no + 1) * (int)gridDim.x - 1) {
                    __hip_atomic_store(sync_flag(sync), no + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                else {
                    const long long t0 = wall_clock64();
                    while (__hip_atomic_load(sync_flag(sync), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) <= no &&
                           wall_clock64() - t0 < spin_ticks)
                        __builtin_amdgcn_s_sleep(1);
                }
            }
        }
        workgroup_barrier();
    }
    if (threadIdx.x == 0) {  // the last workgroup to leave puts the counters back to zero
        const int old = __hip_atomic_fetch_add(sync_done(sync), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (int)gridDim.x - 1) {
            for (int l = 0; l < kLeaves; ++l) __hip_atomic_store(sync_leaf(sync, l), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_root(sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_flag(sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(sync_done(sync), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace

hipError_t launch_probe_barrier(int* sync, int iters, int tree, int cus, long long spin_ticks, hipStream_t st)
{
    if (!sync || iters < 1 || cus < 1) return hipErrorInvalidValue;
    return launch_kernel(barrier_probe_kernel, dim3(cus), dim3(64 * kWaves), 0, st, sync, iters, tree, spin_ticks);
}

bool sequence_feasible(const SeqGemm* g, int count, int T)
{
    if (count < 1 || count > kSeqMax || T < 1 || T > 16) return false;
    for (int i = 0; i < count; ++i) {
        if (g[i].N <= 0 || g[i].K <= 0 || g[i].N % kTileN != 0 || g[i].K % kGroup != 0) return false;
        if ((int64_t)T * g[i].K * 2 >= (1ll << 32)) return false;  // 32-bit lane offsets into X
    }
    return true;
}

int sequence_error_index()
{
    return 64 * (kLeaves + 3);
}

hipError_t sequence_launch(const SeqGemm* g, int count, int T, int* sync, int cus, long long spin_ticks, hipStream_t st)
{
    if (!sequence_feasible(g, count, T) || !sync || cus < 1) return hipErrorInvalidValue;
    SeqArgs a{};
    for (int i = 0; i < count; ++i) a.g[i] = g[i];
    a.count      = count;
    a.T          = T;
    a.sync       = sync;
    a.spin_ticks = spin_ticks;
    const dim3   grid(cus), block(64 * kWaves);
    const int    tp  = T <= 4 ? 4 : (T <= 8 ? 8 : 16);
    const size_t lds = (size_t)kWaves * std::max(kMaxR * 1024, tp * 256);
    if (tp == 4) return launch_kernel(sequence_kernel<4>, grid, block, lds, st, a);
    if (tp == 8) return launch_kernel(sequence_kernel<8>, grid, block, lds, st, a);
    return launch_kernel(sequence_kernel<16>, grid, block, lds, st, a);
}

}  // namespace w4a16
