// Integer repack kernels: AWQ int4 tensors <-> the gfx950 tiled layout, and the other
// nibble permutations of the reference's format.cu.  Every kernel is a pure gather: one
// thread builds one whole destination word from (cached) source words, so no atomics and
// no pre-zeroed destination are needed.
#include "w4a16_common.h"
#include "w4a16_internal.h"

namespace w4a16 {

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ uint32_t nib(uint32_t w, int p)
{
    return (w >> (4 * p)) & 0xfu;
}

// logical column c (0..7) of an AWQ word sits in nibble nibble_of_row(c): the AWQ order and
// its inverse are the same pair of tables that the tiled layout uses along its rows.
__device__ __forceinline__ uint32_t awq_col(uint32_t w, int c)
{
    return nib(w, nibble_of_row(c));
}

__device__ __forceinline__ int64_t global_id()
{
    return (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
}

// A_dst word `w` <- 8 rows of one column of the AWQ matrix.
__global__ void __launch_bounds__(kThreads)
repack_weights_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, int N, int K)
{
    const int64_t w     = global_id();
    const int64_t words = (int64_t)N * K / 8;
    if (w >= words) return;
    const int     NT   = N / kTileN;
    const int     j    = (int)(w & 3);
    const int     lane = (int)((w >> 2) & 63);
    const int64_t tile = w >> 8;
    const int     kt   = (int)(tile / NT);
    const int     nt   = (int)(tile % NT);
    const int     n    = nt * kTileN + (lane & 15);
    const int     k0   = kt * kGroup + 32 * j + 8 * (lane >> 4);
    const int     ld   = N / 8;
    uint32_t      out  = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t s = src[(int64_t)(k0 + e) * ld + (n >> 3)];
        out |= awq_col(s, n & 7) << (4 * nibble_of_row(e));
    }
    dst[w] = out;
}

// Q[g, n] = half2(64 + z, s)
__global__ void __launch_bounds__(kThreads)
merge_q_kernel(uint32_t* __restrict__ Q, const uint16_t* __restrict__ scales,
               const uint32_t* __restrict__ qzeros, int64_t count)
{
    const int64_t i = global_id();
    if (i >= count) return;
    const uint32_t z = awq_col(qzeros[i >> 3], (int)(i & 7));
    Q[i]             = (0x5400u | (z << 4)) | ((uint32_t)scales[i] << 16);
}

// The columns of a deployable matrix, gathered from up to three AWQ tensors of the checkpoint:
// side by side (q | k | v, deploy.py:251-260 `merge_qkv`), optionally with the columns of every
// head re-ordered for rotary embedding (dst column 2i + r of a head <- column r * D/2 + i:
// deploy.py:371-383 `permute`, format.cu:115-121), or interleaved in pairs (gate, up:
// deploy.py:641-658 `fuse_w1_w3_s4`, format.cu:123-130).
struct ColumnSource {
    const uint32_t* qw[3];
    const uint32_t* qz[3];
    const uint16_t* s[3];
    int             width[3];   // columns of each source
    int             rotary[3];  // head size if the block's columns are re-ordered, else 0
    int             interleave; // 1: column n comes from source n & 1, column n >> 1
};
struct Located {
    int src, col;
};
__device__ __forceinline__ Located locate(const ColumnSource& cs, int n)
{
    if (cs.interleave) return Located{n & 1, n >> 1};
    int b = 0;
    while (b < 2 && n >= cs.width[b]) n -= cs.width[b++];
    if (const int D = cs.rotary[b]) {
        const int j = n % D;
        n           = n - j + (j & 1) * (D / 2) + (j >> 1);
    }
    return Located{b, n};
}

// A_dst word `w` <- 8 rows of one column, taken from wherever the column lives
__global__ void __launch_bounds__(kThreads)
deploy_weights_kernel(uint32_t* __restrict__ dst, const ColumnSource cs, int N, int K)
{
    const int64_t w     = global_id();
    const int64_t words = (int64_t)N * K / 8;
    if (w >= words) return;
    const int     NT   = N / kTileN;
    const int     j    = (int)(w & 3);
    const int     lane = (int)((w >> 2) & 63);
    const int64_t tile = w >> 8;
    const int     kt   = (int)(tile / NT);
    const int     nt   = (int)(tile % NT);
    const Located at   = locate(cs, nt * kTileN + (lane & 15));
    const int     k0   = kt * kGroup + 32 * j + 8 * (lane >> 4);
    const int     ld   = cs.width[at.src] / 8;
    const uint32_t* src = cs.qw[at.src];
    uint32_t      out  = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t v = src[(int64_t)(k0 + e) * ld + (at.col >> 3)];
        out |= awq_col(v, at.col & 7) << (4 * nibble_of_row(e));
    }
    dst[w] = out;
}

__global__ void __launch_bounds__(kThreads) deploy_q_kernel(uint32_t* __restrict__ Q, const ColumnSource cs, int N, int G)
{
    const int64_t i = global_id();
    if (i >= (int64_t)N * G) return;
    const int      g  = (int)(i / N);
    const Located  at = locate(cs, (int)(i % N));
    const int64_t  e  = (int64_t)g * cs.width[at.src] + at.col;
    const uint32_t z  = awq_col(cs.qz[at.src][e >> 3], (int)(e & 7));
    Q[i]              = (0x5400u | (z << 4)) | ((uint32_t)cs.s[at.src][e] << 16);
}

// inverse of repack_weights_kernel: one thread per AWQ word [k, n/8]
__global__ void __launch_bounds__(kThreads)
unrepack_weights_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ A, int N, int K)
{
    const int64_t w     = global_id();
    const int64_t words = (int64_t)N * K / 8;
    if (w >= words) return;
    const int ld = N / 8;
    const int k  = (int)(w / ld);
    const int n0 = (int)(w % ld) * 8;
    const int NT = N / kTileN;
    const int kt = k / kGroup, r = k % kGroup;
    const int j = r >> 5, b = (r >> 3) & 3, e = r & 7;
    uint32_t  out = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int     n  = n0 + c;
        const int64_t sw = (((int64_t)kt * NT + n / kTileN) * 64 + b * 16 + (n % kTileN)) * 4 + j;
        out |= nib(A[sw], nibble_of_row(e)) << (4 * nibble_of_row(c));
    }
    dst[w] = out;
}

__global__ void __launch_bounds__(kThreads)
split_q_kernel(uint32_t* __restrict__ qzeros, uint16_t* __restrict__ scales, const uint32_t* __restrict__ Q,
               int64_t words)
{
    const int64_t w = global_id();
    if (w >= words) return;
    uint32_t out = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t q = Q[w * 8 + c];
        out |= ((q >> 4) & 0xfu) << (4 * nibble_of_row(c));
        if (scales) scales[w * 8 + c] = (uint16_t)(q >> 16);
    }
    if (qzeros) qzeros[w] = out;
}

// W[k, n] = mul.ftz(sub(64 + q, 64 + z), s): one thread per repacked word (8 rows of a column)
__global__ void __launch_bounds__(kThreads)
dequantize_repacked_kernel(uint16_t* __restrict__ W, const uint32_t* __restrict__ A,
                           const uint32_t* __restrict__ Q, int N, int K, int group)
{
    const int64_t w     = global_id();
    const int64_t words = (int64_t)N * K / 8;
    if (w >= words) return;
    const int     NT   = N / kTileN;
    const int     j    = (int)(w & 3);
    const int     lane = (int)((w >> 2) & 63);
    const int64_t tile = w >> 8;
    const int     kt   = (int)(tile / NT);
    const int     nt   = (int)(tile % NT);
    const int     n    = nt * kTileN + (lane & 15);
    const int     k0   = kt * kGroup + 32 * j + 8 * (lane >> 4);
    half2_t       z1024, z64;
    half_t        s;
    split_q(Q[(int64_t)(k0 / group) * N + n], z1024, z64, s);  // (a word's 8 rows never straddle two groups: group >= 32)
    // flush a subnormal scale first, as the .ftz multiply of the reference reads it
    uint16_t sb = __builtin_bit_cast(uint16_t, s);
    if ((sb & 0x7c00u) == 0) sb &= 0x8000u;
    s = __builtin_bit_cast(half_t, sb);
    const half8_t v = dequant_full(A[w], z1024, z64, half2_t{s, s}, UnpackConsts());
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        uint16_t bits = __builtin_bit_cast(uint16_t, (half_t)v[e]);
        if ((bits & 0x7c00u) == 0) bits &= 0x8000u;  // flush a subnormal product
        W[(int64_t)(k0 + e) * N + n] = bits;
    }
}

// raw nibble values of AWQ words as fp16, logical column order
__global__ void __launch_bounds__(kThreads)
dequantize_s4_kernel(uint4* __restrict__ dst, const uint32_t* __restrict__ src, int64_t count)
{
    const int64_t i = global_id();
    if (i >= count) return;
    const uint32_t w = src[i];
    uint32_t       v[4];
    unpack_offset(w, v);  // applied to an AWQ word this yields columns (0,1), (2,3), (4,5), (6,7)
    const half2_t k1024 = as_half2(0x64006400u), k64 = as_half2(0x54005400u);
    uint4         o;
    o.x = as_u32(as_half2(v[0]) - k1024);
    o.y = as_u32(as_half2(v[1]) - k64);
    o.z = as_u32(as_half2(v[2]) - k1024);
    o.w = as_u32(as_half2(v[3]) - k64);
    dst[i] = o;
}

// dst AWQ [k, 2m/8] <- interleave of AWQ w1, w3 [2, k, m/8]
__global__ void __launch_bounds__(kThreads)
fuse_w1_w3_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, int m, int k)
{
    const int64_t w     = global_id();
    const int     ldd   = 2 * m / 8;
    const int64_t words = (int64_t)k * ldd;
    if (w >= words) return;
    const int     row = (int)(w / ldd);
    const int     c0  = (int)(w % ldd) * 8;
    const int     lds = m / 8;
    uint32_t      out = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int      col = c0 + c, sel = col & 1, js = col >> 1;
        const uint32_t s   = src[((int64_t)sel * k + row) * lds + (js >> 3)];
        out |= awq_col(s, js & 7) << (4 * nibble_of_row(c));
    }
    dst[w] = out;
}

// within each head of D columns: dst[2i + r] = src[r * D/2 + i]
__global__ void __launch_bounds__(kThreads)
transpose_qk_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src, int m, int k, int D)
{
    const int64_t w     = global_id();
    const int     ld    = m / 8;
    const int64_t words = (int64_t)k * ld;
    if (w >= words) return;
    const int row = (int)(w / ld);
    const int c0  = (int)(w % ld) * 8;
    uint32_t  out = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int      col = c0 + c, h = col / D, ci = col % D;
        const int      sc  = h * D + (ci & 1) * (D / 2) + (ci >> 1);
        const uint32_t s   = src[(int64_t)row * ld + (sc >> 3)];
        out |= awq_col(s, sc & 7) << (4 * nibble_of_row(c));
    }
    dst[w] = out;
}

// ours <- the reference's tiled layout: word ((kt*(N/32)+nt)*32 + lane)*4 + (k16*2 + n16),
// nibble 4*klo + 2*k8 + n8 holds k = 32kt + 16k16 + 8k8 + 2*(lane%4) + klo,
// n = 32nt + 16n16 + 8n8 + lane/4.
__global__ void __launch_bounds__(kThreads)
from_reference_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ ref, int N, int K)
{
    const int64_t w     = global_id();
    const int64_t words = (int64_t)N * K / 8;
    if (w >= words) return;
    const int     NT   = N / kTileN;
    const int     j    = (int)(w & 3);
    const int     lane = (int)((w >> 2) & 63);
    const int64_t tile = w >> 8;
    const int     kt   = (int)(tile / NT);
    const int     nt   = (int)(tile % NT);
    const int     n    = nt * kTileN + (lane & 15);
    const int     k0   = kt * kGroup + 32 * j + 8 * (lane >> 4);
    uint32_t      out  = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int     kk = k0 + e;
        const int     rl = (n & 7) * 4 + ((kk >> 1) & 3);
        const int64_t rw = (((int64_t)(kk >> 5) * (N / 32) + (n >> 5)) * 32 + rl) * 4 + (((kk >> 4) & 1) * 2 + ((n >> 4) & 1));
        const int     rn = 4 * (kk & 1) + 2 * ((kk >> 3) & 1) + ((n >> 3) & 1);
        out |= nib(ref[rw], rn) << (4 * nibble_of_row(e));
    }
    dst[w] = out;
}

inline unsigned blocks_for(int64_t n)
{
    return (unsigned)((n + kThreads - 1) / kThreads);
}

}  // namespace

hipError_t launch_convert(uint32_t* A_dst, uint32_t* Q_dst, const uint32_t* A_src, const uint16_t* scales,
                          const uint32_t* qzeros, int m, int k, int group, hipStream_t st)
{
    const int64_t words = (int64_t)m * k / 8;
    const int64_t qn    = (int64_t)(k / group) * m;
    if (words == 0) return hipSuccess;
    hipError_t e = hipSuccess;
    if (A_dst) e = launch_kernel(repack_weights_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, A_dst, A_src, m, k);
    if (Q_dst && e == hipSuccess)
        e = launch_kernel(merge_q_kernel, dim3(blocks_for(qn)), dim3(kThreads), 0, st, Q_dst, scales, qzeros, qn);
    return e;
}

hipError_t launch_deploy(uint32_t* A_dst, uint32_t* Q_dst, const uint32_t* const qw[3], const uint32_t* const qz[3],
                         const uint16_t* const s[3], const int width[3], const int rotary[3], int interleave, int k,
                         int group, hipStream_t st)
{
    ColumnSource cs{};
    int          m = 0;
    for (int i = 0; i < 3; ++i) {
        cs.qw[i] = qw[i], cs.qz[i] = qz[i], cs.s[i] = s[i];
        cs.width[i] = width[i], cs.rotary[i] = rotary[i];
        m += width[i];
    }
    cs.interleave       = interleave;
    const int64_t words = (int64_t)m * k / 8;
    const int64_t qn    = (int64_t)(k / group) * m;
    if (words == 0) return hipSuccess;
    hipError_t e = launch_kernel(deploy_weights_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, A_dst, cs, m, k);
    if (e == hipSuccess)
        e = launch_kernel(deploy_q_kernel, dim3(blocks_for(qn)), dim3(kThreads), 0, st, Q_dst, cs, m, k / group);
    return e;
}

hipError_t launch_unpack(uint32_t* qweight, uint32_t* qzeros, uint16_t* scales, const uint32_t* A,
                         const uint32_t* Q, int m, int k, int group, hipStream_t st)
{
    const int64_t words = (int64_t)m * k / 8;
    const int64_t qw    = (int64_t)(k / group) * m / 8;
    if (words == 0) return hipSuccess;
    hipError_t e = hipSuccess;
    if (qweight) e = launch_kernel(unrepack_weights_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, qweight, A, m, k);
    if ((qzeros || scales) && e == hipSuccess)
        e = launch_kernel(split_q_kernel, dim3(blocks_for(qw)), dim3(kThreads), 0, st, qzeros, scales, Q, qw);
    return e;
}

hipError_t launch_dequantize_repacked(uint16_t* W, const uint32_t* A, const uint32_t* Q, int m, int k, int group,
                                      hipStream_t st)
{
    const int64_t words = (int64_t)m * k / 8;
    if (words == 0) return hipSuccess;
    return launch_kernel(dequantize_repacked_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, W, A, Q, m, k, group);
}

hipError_t launch_dequantize_s4(void* dst, const uint32_t* src, size_t count, hipStream_t st)
{
    if (count == 0) return hipSuccess;
    return launch_kernel(dequantize_s4_kernel, dim3(blocks_for((int64_t)count)), dim3(kThreads), 0, st, (uint4*)dst,
                         src, (int64_t)count);
}

hipError_t launch_fuse_w1_w3(uint32_t* dst, const uint32_t* src, int m, int k, hipStream_t st)
{
    const int64_t words = (int64_t)k * (2 * m / 8);
    if (words == 0) return hipSuccess;
    return launch_kernel(fuse_w1_w3_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, dst, src, m, k);
}

hipError_t launch_transpose_qk(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head, hipStream_t st)
{
    const int64_t words = (int64_t)k * (m / 8);
    if (words == 0) return hipSuccess;
    return launch_kernel(transpose_qk_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, dst, src, m, k,
                         size_per_head);
}

hipError_t launch_from_reference(uint32_t* dst, const uint32_t* ref, int m, int k, hipStream_t st)
{
    const int64_t words = (int64_t)m * k / 8;
    if (words == 0) return hipSuccess;
    return launch_kernel(from_reference_kernel, dim3(blocks_for(words)), dim3(kThreads), 0, st, dst, ref, m, k);
}

}  // namespace w4a16
