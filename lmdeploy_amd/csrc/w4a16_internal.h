// Internal C++ interface between the C ABI (api.hip) and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace w4a16 {

enum Epilogue { kEpiGemm = 0, kEpiSilu = 1, kEpiAdd = 2 };

struct GemmArgs {
    uint16_t*       C;   // fp16 out [T, N] or [T, N/2]
    const uint32_t* A;   // tiled int4 weights
    const uint16_t* X;   // fp16 [T, K]
    const uint32_t* Q;   // half2 [K/128, N]
    const uint16_t* R;   // fp16 residual [T, N] or null
    int             N, T, K;
    int             epilogue;
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

// Scratch owned by a handle: split-K partial tiles and arrival counters.  Every handle has exactly
// this much, so feasibility of a split-K launch does not depend on the handle.
constexpr size_t kWorkspaceBytes = 64u << 20;
constexpr int    kCounters       = 1 << 16;
struct Scratch {
    float* ws;
    size_t ws_bytes;
    int*   cnt;
    int    cnt_len;
};

int         algo_count();
const Algo& algo_at(int id);
// true if algo `id` can run the shape
bool algo_feasible(int id, int N, int T, int K);
// heuristic choice (the counterpart of Estimate); -1 if nothing is feasible
int algo_pick(int N, int T, int K);
// workgroups the launch would use
int algo_grid(int id, int N, int T, int K, const Scratch& sc);
hipError_t algo_launch(int id, const GemmArgs& a, const Scratch& sc, hipStream_t st);

hipError_t launch_convert(uint32_t* A_dst, uint32_t* Q_dst, const uint32_t* A_src, const uint16_t* scales,
                          const uint32_t* qzeros, int m, int k, hipStream_t st);
hipError_t launch_unpack(uint32_t* qweight, uint32_t* qzeros, uint16_t* scales, const uint32_t* A,
                         const uint32_t* Q, int m, int k, hipStream_t st);
hipError_t launch_dequantize_repacked(uint16_t* W, const uint32_t* A, const uint32_t* Q, int m, int k,
                                      hipStream_t st);
hipError_t launch_dequantize_s4(void* dst, const uint32_t* src, size_t count, hipStream_t st);
hipError_t launch_fuse_w1_w3(uint32_t* dst, const uint32_t* src, int m, int k, hipStream_t st);
hipError_t launch_transpose_qk(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head, hipStream_t st);
hipError_t launch_from_reference(uint32_t* dst, const uint32_t* ref, int m, int k, hipStream_t st);

// decode (skinny) kernels
bool       decode_feasible(const DecodeConfig& cf, int N, int T, int K);
int        decode_grid(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len);
hipError_t decode_launch(const DecodeConfig& cf, const GemmArgs& a, float* ws, size_t ws_bytes, int* cnt, int cnt_len,
                         hipStream_t st);

// decode kernels, strip decomposition (gemm_strip.hip); block_t = tokens per workgroup, 16 or 32
bool       strip_feasible(int per_cu, int block_t, int N, int T, int K);
int        strip_grid(int per_cu, int block_t, int N, int T, int K);
int        strip_width(int per_cu, int block_t, int N, int T, int K);  // column tiles of the widest strip
hipError_t strip_launch(int per_cu, int block_t, const GemmArgs& a, hipStream_t st);

// MFMA prefill kernels
int        prefill_variants();
void       prefill_tile(int variant, int& tile_n, int& tile_t);
// `splits` > 1 divides the quantisation groups among that many workgroups per output tile; the
// last one to arrive adds the partial tiles (in split order) and runs the epilogue.
bool       prefill_feasible(int variant, int splits, int N, int T, int K);
int        prefill_grid(int variant, int splits, int N, int T, int K);
hipError_t prefill_launch(int variant, int splits, const GemmArgs& a, const Scratch& sc, hipStream_t st);
double     prefill_estimate_us(int variant, int splits, int N, int T, int K);  // model fitted to measurements

}  // namespace w4a16
