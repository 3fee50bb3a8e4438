// Internal C++ interface between the C ABI (api.cpp) and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>

namespace w4a16 {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

enum Epilogue { kEpiGemm = 0, kEpiSilu = 1, kEpiAdd = 2 };

struct GemmArgs {
    uint16_t*       C;   // fp16 out [T, N] or [T, N/2]
    const uint32_t* A;   // tiled int4 weights
    const uint16_t* X;   // fp16 [T, K]
    const uint32_t* Q;   // half2 [K/128, N]
    const uint16_t* R;   // fp16 residual [T, N] or null
    int             N, T, K;
    int             epilogue;
    unsigned long long* clk = nullptr;  // measurement aid: where a strip kernel adds its cycle and tick counts (3 words)
};

// One dispatchable kernel configuration.
// A decode kernel configuration: r column tiles per wave, wn waves per slice, sk slices per
// workgroup, `depth` groups of weights in flight per wave; fill > 0 additionally splits K
// across workgroups until about `fill` workgroups per CU exist.
struct DecodeConfig {
    int r, wn, sk, depth, fill;
};

struct Algo {
    int          kind;     // 0 decode (column blocks), 1 prefill, 2 decode (strips)
    int          tile_n;   // output features per workgroup
    int          tile_t;   // tokens per workgroup
    int          slices;   // decode: K slices per workgroup; prefill: K splits across workgroups
    int          param;    // prefill: variant index; strips: strips per CU aimed for
    DecodeConfig dc;       // decode only
};

// Scratch of the split-K kernels: fp32 partial tiles and arrival counters.  A handle's scratch has
// exactly this size (the partial tiles are allocated on first need, the counters with the handle),
// so feasibility of a split-K launch does not depend on the handle.  `ws_bytes` / `cnt_len` say
// how much a launch may use; `ws` may still be null while they are non-zero (not yet allocated).
constexpr size_t kWorkspaceBytes = 64u << 20;
constexpr int    kCounters       = 1 << 16;
struct Scratch {
    float* ws;
    size_t ws_bytes;
    int*   cnt;
    int    cnt_len;
};

// Launches `kernel` and returns this launch's own status.  (The triple-chevron form reports through
// hipGetLastError, which also returns - and clears - an error some earlier call of the caller left behind.)
template<typename... P, typename... A>
inline hipError_t launch_kernel(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t st, A... args)
{
    std::tuple<P...> held{static_cast<P>(args)...};
    void*            ptrs[sizeof...(P) > 0 ? sizeof...(P) : 1];
    int              i = 0;
    std::apply([&](auto&... v) { ((ptrs[i++] = (void*)&v), ...); }, held);
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds, st);
}

// Raises a kernel's dynamic LDS limit once per kernel instantiation (`done`: one bit per device) and
// device; kernels that ask for more than 64 KiB need it before their first launch on a device.
inline hipError_t raise_lds_limit(const void* kernel, int bytes, std::atomic<uint64_t>& done)
{
    int        dev = 0;
    hipError_t e   = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

int         algo_count();
const Algo& algo_at(int id);
// true if algo `id` can run the shape with the scratch `lim` allows
bool algo_feasible(int id, int N, int T, int K, const Scratch& lim);
// bytes of partial-tile scratch the launch would use (0: the kernel needs neither workspace nor counters)
size_t algo_scratch_bytes(int id, int N, int T, int K, const Scratch& lim);
// heuristic choice (the counterpart of Estimate); -1 if nothing is feasible
int algo_pick(int N, int T, int K, const Scratch& lim);
// workgroups the launch would use
int algo_grid(int id, int N, int T, int K, const Scratch& sc);
hipError_t algo_launch(int id, const GemmArgs& a, const Scratch& sc, hipStream_t st);

// The scratch that lives in a file-scope device array (static_scratch.hip), for callers that cannot
// allocate: its address on the current device, looked up once per device.
constexpr size_t kStaticCounters       = 4096;
constexpr size_t kStaticWorkspaceBytes = 8u << 20;
hipError_t static_scratch(Scratch* out);
// zeroes the first `n` arrival counters of `sc` with a fill kernel on `st`
hipError_t clear_counters(const Scratch& sc, int n, hipStream_t st);

hipError_t launch_convert(uint32_t* A_dst, uint32_t* Q_dst, const uint32_t* A_src, const uint16_t* scales,
                          const uint32_t* qzeros, int m, int k, int group, hipStream_t st);
// up to three AWQ tensors -> one deployable (A, Q): side by side, or (interleave) gate/up column pairs
hipError_t launch_deploy(uint32_t* A_dst, uint32_t* Q_dst, const uint32_t* const qw[3], const uint32_t* const qz[3],
                         const uint16_t* const s[3], const int width[3], const int rotary[3], int interleave, int k,
                         int group, hipStream_t st);
hipError_t launch_unpack(uint32_t* qweight, uint32_t* qzeros, uint16_t* scales, const uint32_t* A,
                         const uint32_t* Q, int m, int k, int group, hipStream_t st);
hipError_t launch_dequantize_repacked(uint16_t* W, const uint32_t* A, const uint32_t* Q, int m, int k, int group,
                                      hipStream_t st);
hipError_t launch_dequantize_s4(void* dst, const uint32_t* src, size_t count, hipStream_t st);
hipError_t launch_fuse_w1_w3(uint32_t* dst, const uint32_t* src, int m, int k, hipStream_t st);
hipError_t launch_transpose_qk(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head, hipStream_t st);
hipError_t launch_from_reference(uint32_t* dst, const uint32_t* ref, int m, int k, hipStream_t st);

// measurement aid (probe.hip): a plain streaming read of `bytes`; sink = at least 8 * cus words
hipError_t launch_probe_read(const void* src, size_t bytes, void* sink, int cus, hipStream_t st);
// the same with the GEMM kernels' load pipeline: `in_flight` (2, 4, 8, 16) loads of 16 bytes per lane kept in
// flight by count, `wg_per_cu` (1, 2, 4) workgroups of eight waves per CU, hint 0 none / 1 nt / 2 sc0 sc1
bool       probe_stream_config_ok(int wg_per_cu, int in_flight, int hint);
// (clk: optional counters of clock_record_start / _stop)
hipError_t launch_probe_mfma(void* sink, int cus, int waves_per_cu, int iters, unsigned long long* clk, hipStream_t st);
hipError_t launch_probe_stream(const void* src, size_t bytes, void* sink, int cus, int wg_per_cu, int in_flight, int hint,
                               hipStream_t st, unsigned long long* clk = nullptr);

// decode (skinny) kernels
bool       decode_feasible(const DecodeConfig& cf, int N, int T, int K);
size_t     decode_scratch_bytes(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len);
int        decode_grid(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len);
hipError_t decode_launch(const DecodeConfig& cf, const GemmArgs& a, float* ws, size_t ws_bytes, int* cnt, int cnt_len,
                         hipStream_t st);

// decode kernels, strip decomposition (gemm_strip.hip); block_t = tokens per workgroup, 16 or 32
bool       strip_feasible(int per_cu, int block_t, int N, int T, int K);
int        strip_grid(int per_cu, int block_t, int N, int T, int K);
int        strip_width(int per_cu, int block_t, int N, int T, int K);  // column tiles of the widest strip
hipError_t strip_launch(int per_cu, int block_t, const GemmArgs& a, hipStream_t st);
// the strip kernel for group sizes 64 and 32 (nq = 2, 4 quantisation groups per 128-row weight tile), any token count
bool       strip_groups_feasible(int nq, int N, int T, int K);
hipError_t strip_groups_launch(int nq, const GemmArgs& a, hipStream_t st);

// A sequence of decode GEMMs (up to 16 tokens) in one persistent launch (gemm_sequence.hip)
struct SeqGemm {
    uint16_t*       C;
    const u32x4_t*  A;
    const uint16_t* X;
    const uint32_t* Q;
    const uint16_t* R;
    int             N, K;
    int             epilogue;
    int             flags;  // bit 0: reads what an earlier GEMM of the sequence writes - wait for all of them
};
constexpr int kSeqMax   = 32;    // GEMMs per launch (the descriptors travel as kernel arguments)
constexpr int kSyncInts = 64 * 80;  // arrival counters, flag, error word of the device-wide barrier
bool       sequence_feasible(const SeqGemm* g, int count, int T);
int        sequence_error_index();  // index of the error word in the sync area
// `cus` workgroups (one per CU: they must all be resident at once); `spin_ticks` bounds each barrier wait
hipError_t sequence_launch(const SeqGemm* g, int count, int T, int* sync, int cus, long long spin_ticks, hipStream_t st);

// measurement aid: `iters` device-wide barriers of `cus` workgroups (tree = 0: all arrivals on one counter)
hipError_t launch_probe_barrier(int* sync, int iters, int tree, int cus, long long spin_ticks, hipStream_t st);

// MFMA prefill kernels
int        prefill_variants();
void       prefill_tile(int variant, int& tile_n, int& tile_t);
// `splits` > 1 divides the quantisation groups among that many workgroups per output tile; the
// last one to arrive adds the partial tiles (in split order) and runs the epilogue.
bool       prefill_feasible(int variant, int splits, int N, int T, int K, size_t ws_bytes, int cnt_len);
size_t     prefill_scratch_bytes(int variant, int splits, int N, int T, int K);
int        prefill_grid(int variant, int splits, int N, int T, int K);
hipError_t prefill_launch(int variant, int splits, const GemmArgs& a, const Scratch& sc, hipStream_t st);
double     prefill_estimate_us(int variant, int splits, int N, int T, int K);  // model fitted to measurements
// the 256 x 128 prefill tile for group sizes 64 and 32 (nq = 2, 4); needs n_out % 128 == 0
bool       prefill_groups_feasible(int nq, int N, int T, int K);
hipError_t prefill_groups_launch(int nq, const GemmArgs& a, hipStream_t st);

}  // namespace w4a16
