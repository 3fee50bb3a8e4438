// The strip decomposition of the decode (skinny) W4A16 GEMM for gfx950, shared by the one-GEMM
// kernel (gemm_strip.hip) and the persistent kernel that runs a sequence of GEMMs in one launch
// (gemm_sequence.hip).
//
// The weight matrix is a grid of 1 KiB tiles (16 columns x one 128-row quantisation group).  The
// column tiles are dealt out as evenly as possible to B workgroups: workgroup b owns a strip of R or
// R-1 adjacent column tiles over the whole of K.  Its eight waves deal the groups of K out
// round-robin; a wave walks its groups and, per group, loads the strip's R tiles (R KiB contiguous
// in the group-major tile layout) and its own activations of that group straight into registers -
// no cooperative staging, no barrier and no other wave involved until the end, when the eight
// partial strips are added in LDS in slice order.
#pragma once

#include "w4a16_common.h"
#include "w4a16_internal.h"

#include <type_traits>

namespace w4a16 {

namespace strip {

constexpr int kWaves   = 8;  // = K slices per workgroup
constexpr int kMaxR    = 8;  // column tiles per strip
constexpr int kMaxR32  = 8;  // ... with 32 tokens per workgroup
constexpr int kNumCU   = 256;  // MI355X; the deal itself asks the device (gemm_strip.hip)
constexpr int kDmaTokens = 32;  // token block from which the activations go straight to LDS

struct StripParams {
    uint16_t*       C;
    const u32x4_t*  A;
    const uint16_t* X;
    const uint32_t* Q;
    const uint16_t* Rsd;
    int             N, T, K;
    int             base;  // column tiles of a narrow strip
    int             rem;   // the first `rem` strips have base + 1
    int             epilogue;  // read by kernels whose epilogue is chosen at run time (EPI == kEpiRuntime)
    int             passes;    // strips per workgroup, one after the other (strip number = pass * workgroups + workgroup)
    unsigned long long* clk = nullptr;  // measurement aid (clock_record_start / _stop); null in every ordinary launch
};

constexpr int kEpiRuntime = 3;  // template value: take the epilogue from StripParams

// Loads of the software pipeline: issued from inline assembly, in place ("+v"), with a scalar
// base, a per-lane 32-bit offset and an immediate, and waited for by count (the compiler would
// drain every load in flight at the loop header).  `LOADS(...)` wraps a few of them in an EXEC
// mask: with flag 0 the instructions still issue and still count in vmcnt, but touch neither
// memory nor their destination, which lets the last trips of a loop skip their refills without
// a branch - the number of loads in flight stays a compile-time constant.
#define W4A16_MASKED(body)                                                                                             \
    "s_mov_b64 %[sv], exec\n\ts_cmp_lg_u32 %[mk], 0\n\ts_cselect_b64 exec, exec, 0\n\t" body "s_mov_b64 exec, %[sv]"

template<int IM>
__device__ __forceinline__ void mload32(uint32_t& dst, uint32_t voff, const void* sbase, int flag)
{
    uint64_t sv;
    asm volatile(W4A16_MASKED("global_load_dword %[d], %[vo], %[sb] offset:%[im]\n\t")
                 : [d] "+v"(dst), [sv] "=&s"(sv)
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag), [im] "n"(IM)
                 : "scc");
}
template<int IM>
__device__ __forceinline__ void mload128_nt(u32x4_t& dst, uint32_t voff, const void* sbase, int flag)
{
    uint64_t sv;
    asm volatile(W4A16_MASKED("global_load_dwordx4 %[d], %[vo], %[sb] offset:%[im] nt\n\t")
                 : [d] "+v"(dst), [sv] "=&s"(sv)
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag), [im] "n"(IM)
                 : "scc");
}
__device__ __forceinline__ void mload128(u32x4_t& dst, uint32_t voff, const void* sbase, int flag)
{
    uint64_t sv;
    asm volatile(W4A16_MASKED("global_load_dwordx4 %[d], %[vo], %[sb]\n\t")
                 : [d] "+v"(dst), [sv] "=&s"(sv)
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag)
                 : "scc");
}
// the same at agent scope: for data that another workgroup of the same launch, possibly on another
// XCD (each XCD has its own L2), has written with agent-scope stores
__device__ __forceinline__ void mload128_agent(u32x4_t& dst, uint32_t voff, const void* sbase, int flag)
{
    uint64_t sv;
    asm volatile(W4A16_MASKED("global_load_dwordx4 %[d], %[vo], %[sb] sc1\n\t")
                 : [d] "+v"(dst), [sv] "=&s"(sv)
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag)
                 : "scc");
}

// Global memory straight into LDS (no registers): lane l's 16 bytes land at lds_base + 16 l.  The LDS
// base travels in M0.  Counts in vmcnt like any other load, and is complete there when the data is in LDS.
__device__ __forceinline__ uint32_t lds_addr(const void* p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(p);
}
__device__ __forceinline__ void mload128_lds(uint32_t lds_base, uint32_t voff, const void* sbase, int flag)
{
    uint64_t sv;
    asm volatile("s_mov_b32 m0, %[lb]\n\t" W4A16_MASKED("global_load_lds_dwordx4 %[vo], %[sb]\n\t")
                 : [sv] "=&s"(sv)
                 : [vo] "v"(voff), [sb] "s"(sbase), [mk] "s"(flag), [lb] "s"(lds_base)
                 : "scc", "m0", "memory");
}
// LDS fragment read from inline assembly: the compiler would put a wait for every load in flight in front of
// an LDS read of its own that follows a direct-to-LDS load.
template<int OFF>
__device__ __forceinline__ void lds_read128(half8_t& dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

template<int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Everything one wave holds for one group: R weight tiles, their Q words, and the activations of
// the group (NX loads of four token rows x 256 bytes each, one 16-byte chunk per lane).
// NQ = quantisation groups per weight tile: 1 (group size 128), 2 (64) or 4 (32); tile r's words are q[r * NQ ..].
template<int R, int NX, int NQ = 1>
struct Stage {
    u32x4_t  w[R];
    uint32_t q[R * NQ];
    u32x4_t  x[NX > 0 ? NX : 1];  // (NX = 0: the activations go straight to LDS)
};

// The whole kernel for a strip of exactly R column tiles starting at tile `col0`.
// SEQ: the GEMM is one of a sequence inside a persistent launch.  Its activations and residual may
// have been written by other workgroups of the same launch, so they are read at agent scope, and its
// output is written at agent scope (write-through) for the same reason; the token block is 0.  The
// weights and (scale, zero) words of the first groups are requested at once; `inputs_ready()` is then
// called by every wave (it returns, workgroup-wide, when activations and residual may be read and LDS
// may be overwritten) before anything else is touched.
struct NoWait {
    __device__ __forceinline__ void operator()() const {}
};
// NW = waves of the workgroup = slices of K.
// NQ: quantisation groups per 128-row weight tile (group sizes 128, 64, 32 = NQ 1, 2, 4).  The weight layout does
// not depend on it; Q then has NQ rows per tile row, and every 128 / NQ rows of a tile have their own scale and
// zero point: NQ shorter MFMA chains per tile, each scaled into the accumulator by itself.
// DD: groups in flight per wave.  Two, unless the strip is so wide that two groups of it from every wave of the CU
// are more than the memory system takes at once (the launcher decides); then one.
template<int R, int TP, int EPI, bool SEQ = false, int NW = kWaves, typename Ready = NoWait, int NQ = 1, int DD = 2>
__device__ __forceinline__ void strip_body(const StripParams& p, int col0, u32x4_t* smem, Ready&& inputs_ready = Ready{})
{
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c    = lane & 15;
    const int b    = lane >> 4;
    const int N = p.N, T = p.T, K = p.K;
    const int G  = K / kGroup;
    const int NT = N / kTileN;
    // H row blocks of 16 tokens share every unpacked weight (H = 2 for the 32-token variant)
    constexpr int H  = TP > 16 ? TP / 16 : 1;
    const int     t0 = SEQ ? 0 : blockIdx.y * (16 * H);
    const int     Tl = min(16 * H, T - t0);

    // this wave's groups: wave, wave + 8, wave + 16, ...  Interleaved rather than blocked, so that
    // at any moment the whole chip reads one contiguous run of a few dozen group rows of the
    // group-major weight array instead of eight distant ones (measured: DRAM prefers that).
    const int g0  = wave;
    const int cnt = (G - wave + NW - 1) / NW;  // 0 if wave >= G
    constexpr int kStep = NW;
    // per-lane byte offsets; everything that depends on the group is scalar
    const uint32_t w_off = (uint32_t)(lane * 16);                    // + (g * NT + col0 + r) * 1024
    const uint32_t q_off = (uint32_t)(c * 4);                        // + (g * N + (col0 + r) * 16) * 4
    // Activations: load i of a group fetches token rows 4i .. 4i+3, lane l the 16-byte chunk l % 16
    // of row 4i + l / 16 - a quarter wave reads one contiguous 256-byte row, two cache lines.
    // (Fetching straight in MFMA operand order, lane (c, b) = row c, makes every quarter wave
    // touch 16 rows; the cache looks up one line per row and request, and at 16 tokens that cost
    // more than the weight stream.)  The wave turns the rows into operand order through a private
    // patch of LDS; chunk p of row r sits at position p ^ r so that both the row-wise writes and
    // the column-wise reads are free of bank conflicts.
    // With 32 tokens the rows go from global memory straight into the patch instead (no registers, no
    // LDS write), one patch per group in flight; the swizzle is then applied on the way in: the lane
    // that lands at position p of row r fetches chunk p ^ r.
    constexpr int  D    = DD;  // groups in flight per wave
    static_assert(D == 2 || (D == 1 && !SEQ), "one or two groups in flight");
    constexpr bool XDMA = TP >= kDmaTokens && !SEQ;
    constexpr int  NX   = TP / 4;
    constexpr int  NXR  = XDMA ? 0 : NX;  // activation loads that land in registers
    uint32_t       x_off[NX];
#pragma unroll
    for (int i = 0; i < NX; ++i) {
        const int r     = 4 * i + (lane >> 4);
        const int chunk = XDMA ? ((lane & 15) ^ (r & 15)) : (lane & 15);
        x_off[i]        = (uint32_t)min(t0 + r, T - 1) * (uint32_t)(K * 2) + (uint32_t)(chunk * 16);
    }
    u32x4_t* const xw = smem + wave * (TP * 16) * (XDMA ? D : 1);  // this wave's patch(es): [TP rows][16 chunks]
    const uint32_t xw_lds = __builtin_amdgcn_readfirstlane(lds_addr(xw));
    int            xw_at[NX], xr_at[H][4];
#pragma unroll
    for (int i = 0; i < NX; ++i) {
        const int r = 4 * i + (lane >> 4);
        xw_at[i]    = r * 16 + ((lane & 15) ^ (r & 15));
    }
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 16 * h + (c & (TP - 1));  // MFMA rows >= TP repeat a lower row: they only feed outputs that are never stored
            xr_at[h][j] = r * 16 + ((4 * j + b) ^ (r & 15));
        }

    const char* Ab = reinterpret_cast<const char*>(p.A) + (int64_t)col0 * 1024;
    const char* Qb = reinterpret_cast<const char*>(p.Q) + (int64_t)col0 * 64;
    const char* Xb = reinterpret_cast<const char*>(p.X);

    // All loads of group g into stage s (number d); enable = false turns them into no-ops that still count.
    using StageT = Stage<R, NXR, NQ>;
    static_assert(NQ == 1 || NQ == 2 || NQ == 4, "group sizes 128, 64 and 32");
    auto issue_x = [&](StageT& s, int d, int g, bool enable) {
        const int flag = __builtin_amdgcn_readfirstlane(enable ? 1 : 0);
        static_for<0, NX>([&](auto i) {
            if constexpr (XDMA) mload128_lds(xw_lds + (uint32_t)(d * TP * 256 + i * 1024), x_off[i], Xb + (int64_t)g * 256, flag);
            else if constexpr (SEQ) mload128_agent(s.x[i], x_off[i], Xb + (int64_t)g * 256, flag);
            else mload128(s.x[i], x_off[i], Xb + (int64_t)g * 256, flag);
        });
    };
    auto issue_wq = [&](StageT& s, int g, bool enable) {
        const int flag = __builtin_amdgcn_readfirstlane(enable ? 1 : 0);
        static_for<0, NQ>([&](auto sub) {
            const char* qg = Qb + ((int64_t)g * NQ + sub) * N * 4;
            static_for<0, R>([&](auto r) { mload32<r * 64>(s.q[r * NQ + sub], q_off, qg, flag); });
        });
        // the tiles of a group are contiguous; immediates reach 4 KiB, so every fourth tile gets a new base
        static_for<0, R>([&](auto r) {
            const char* wg = Ab + ((int64_t)g * NT + (r / 4) * 4) * 1024;
            mload128_nt<(r % 4) * 1024>(s.w[r], w_off, wg, flag);
        });
    };
    auto issue = [&](StageT& s, int d, int g, bool enable) {
        issue_x(s, d, g, enable);
        issue_wq(s, g, enable);
    };
    constexpr int kLoads = R + R * NQ + NX;  // loads per stage

    const UnpackConsts uc;
    // B operand of the chain that sums the activations: -(unpack offset) in columns 0-7, -1 in columns 8-15
    half8_t bsum;
    {
        const half_t lo = c < 8 ? (half_t)-1024.f : (half_t)-1.f, hi = c < 8 ? (half_t)-64.f : (half_t)-1.f;
        bsum = half8_t{lo, lo, hi, hi, lo, lo, hi, hi};
    }
    float4_t           acc[H][R];
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[h][r] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One tile of one group.  U tiles are worked on at a time with their MFMA chains interleaved:
    // a chain is four or eight dependent MFMAs, and a dependent MFMA cannot issue before its predecessor
    // has left the pipe.
    auto compute = [&](StageT& s, auto dc) {
        half8_t xf[H][4];
        if constexpr (XDMA) {
            // the group's rows are in patch d: row block h is 4 KiB further on
            constexpr int d = decltype(dc)::value;
            static_for<0, H * 4>([&](auto hj) {
                constexpr int h = decltype(hj)::value / 4, j = decltype(hj)::value % 4;
                lds_read128<d * TP * 256 + h * 4096>(xf[h][j], xw_lds + (uint32_t)(xr_at[0][j] * 16));
            });
            // (every fragment exactly once: a register named twice would be copied before the wait)
            static_assert(H <= 2, "the wait below names the fragments of at most two row blocks");
            if constexpr (H == 1)
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xf[0][0]), "+v"(xf[0][1]), "+v"(xf[0][2]), "+v"(xf[0][3]));
            else
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(xf[0][0]), "+v"(xf[0][1]), "+v"(xf[0][2]), "+v"(xf[0][3]), "+v"(xf[H - 1][0]),
                               "+v"(xf[H - 1][1]), "+v"(xf[H - 1][2]), "+v"(xf[H - 1][3]));
        }
        else {
#pragma unroll
            for (int i = 0; i < NXR; ++i) xw[xw_at[i]] = s.x[i];
#pragma unroll
            for (int h = 0; h < H; ++h)
#pragma unroll
                for (int j = 0; j < 4; ++j) xf[h][j] = __builtin_bit_cast(half8_t, xw[xr_at[h][j]]);  // same wave: LDS keeps the order
        }
        constexpr int U  = 2;
        constexpr int JN = 4 / NQ;  // k32 chunks per quantisation group
        // What the unpack offsets and the zero points add to every dot product depends on the weights only
        // through z: sum x (q + o) - P - z S = sum x (q - z) with P = sum o x (o = 1024 under the low-nibble
        // pairs, 64 under the high ones) and S = sum x.  A strip of two or more tiles takes P and S from one
        // MFMA chain per quantisation group (columns 0-7 of its B operand hold -o, columns 8-15 hold -1) and
        // every tile starts its own chain from -P: four MFMAs per tile instead of eight.  A strip of one tile
        // runs the second chain per tile, with -(o + z) as its B operand; that costs it no more MFMAs and
        // saves the exchange between the two halves of the columns.
        constexpr bool kSums = R >= 2;
#pragma unroll
        for (int sub = 0; sub < NQ; ++sub) {  // the rows of the tiles that share a scale and a zero point
            float4_t nP[H], nS[H];
            if constexpr (kSums) {
#pragma unroll
                for (int h = 0; h < H; ++h) {
                    float4_t ps = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = sub * JN; j < (sub + 1) * JN; ++j)
                        ps = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[h][j], bsum, ps, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        // the lane eight columns away, row_ror:8 (source given as the old value too: with a constant
                        // there the compiler merges the four moves into one)
                        const int   mine  = __builtin_bit_cast(int, (float)ps[i]);
                        const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(mine, mine, 0x128, 0xf, 0xf, false));
                        nP[h][i] = c < 8 ? ps[i] : other;
                        nS[h][i] = c < 8 ? other : ps[i];
                    }
                }
            }
#pragma unroll
            for (int r0 = 0; r0 < R; r0 += U) {
                float4_t g4[H][U];
                float    sf[U], zf[U];
                half8_t  bz[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int      r  = r0 + u < R ? r0 + u : R - 1;
                    const uint32_t qw = s.q[r * NQ + sub];  // half2(64 + z, scale): z is bits 4-7
                    const half2_t  h2 = as_half2(qw);
                    if constexpr (kSums) {
                        zf[u] = (float)((qw >> 4) & 0xfu);
                        asm volatile("" : "+v"(zf[u]));
                    }
                    else {
                        // -(1024 + z) under the low-nibble pairs, -(64 + z) under the high-nibble pairs
                        const half2_t  n64 = half2_t{h2[0], h2[0]} * half2_t{(half_t)-1.f, (half_t)-1.f};
                        const uint32_t zb  = ((qw >> 4) & 0xfu) * 0x10001u + 0xE400E400u;  // -(1024 + z) twice
                        bz[u][0] = as_half2(zb)[0]; bz[u][1] = as_half2(zb)[1]; bz[u][2] = n64[0]; bz[u][3] = n64[1];
                        bz[u][4] = bz[u][0]; bz[u][5] = bz[u][1]; bz[u][6] = bz[u][2]; bz[u][7] = bz[u][3];
                    }
                    // Convert the scale now and hide it from the optimiser: otherwise the conversion is
                    // folded into the final multiply-add, the Q word stays live past the refill of this
                    // stage, and the refill lands in a copy that is moved back while still in flight.
                    sf[u] = scale_is_normal(qw) ? (float)h2[1] : 0.f;
                    asm volatile("" : "+v"(sf[u]));
#pragma unroll
                    for (int h = 0; h < H; ++h) {
                        if constexpr (kSums) g4[h][u] = nP[h];
                        else g4[h][u] = float4_t{0.f, 0.f, 0.f, 0.f};
                    }
                }
                if constexpr (!kSums) {
#pragma unroll
                    for (int j = sub * JN; j < (sub + 1) * JN; ++j) {
#pragma unroll
                        for (int u = 0; u < U; ++u)
#pragma unroll
                            for (int h = 0; h < H; ++h)
                                if (r0 + u < R) g4[h][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[h][j], bz[u], g4[h][u], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int j = sub * JN; j < (sub + 1) * JN; ++j) {
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        if (r0 + u < R) {
                            uint32_t v[4];
                            unpack_offset(s.w[r0 + u][j], v, uc);
                            half8_t wf;
                            wf[0] = as_half2(v[0])[0]; wf[1] = as_half2(v[0])[1]; wf[2] = as_half2(v[1])[0]; wf[3] = as_half2(v[1])[1];
                            wf[4] = as_half2(v[2])[0]; wf[5] = as_half2(v[2])[1]; wf[6] = as_half2(v[3])[0]; wf[7] = as_half2(v[3])[1];
#pragma unroll
                            for (int h = 0; h < H; ++h)
                                g4[h][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[h][j], wf, g4[h][u], 0, 0, 0);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int h = 0; h < H; ++h)
                        if (r0 + u < R) {
                            if constexpr (kSums) acc[h][r0 + u] += sf[u] * (g4[h][u] + zf[u] * nS[h]);
                            else acc[h][r0 + u] += sf[u] * g4[h][u];
                        }
            }
        }
    };
    // Wait until the stage's loads are complete (loads return in order: at most `kLoads` younger
    // ones may still be in flight, or none after the last issue), then pin its registers below
    // the wait.
    auto pin = [&](StageT& s) {
#pragma unroll
        for (int r = 0; r < R; ++r) asm volatile("" : "+v"(s.w[r]));
#pragma unroll
        for (int r = 0; r < R * NQ; ++r) asm volatile("" : "+v"(s.q[r]));
#pragma unroll
        for (int i = 0; i < NXR; ++i) asm volatile("" : "+v"(s.x[i]));
    };
    // Two groups in flight per wave.  (Three or four fit the register file for narrow strips but
    // measured slower: the unrolled loop body grows with D and is executed only once or twice.)
    static_assert((D - 1) * kLoads <= 63, "vmcnt is a 6-bit counter");
    StageT st[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
#pragma unroll
        for (int r = 0; r < R; ++r) st[d].w[r] = u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int r = 0; r < R * NQ; ++r) st[d].q[r] = 0;
#pragma unroll
        for (int i = 0; i < NXR; ++i) st[d].x[i] = u32x4_t{0, 0, 0, 0};
    }

    // One group: wait for the stage (exactly D - 1 younger stages are in flight behind it), use
    // it, refill it.  Nothing of a stage may be live when it is refilled (the refill is in place
    // and asynchronous), so the scheduler must not move the stage's arithmetic below its refill.
    auto step = [&](auto dc, bool use, int refill_group, bool refill) {
        constexpr int d = decltype(dc)::value;
        StageT&       s = st[d];
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 1) * kLoads) : "memory");
        pin(s);
        if (use) compute(s, dc);
        __builtin_amdgcn_sched_barrier(0);
        issue(s, d, min(refill_group, G - 1), refill);
    };

    if constexpr (SEQ) {
        // weights first (they depend on nothing), then wait for the producers of the activations, then the
        // activations; all of it complete before the loop, whose counted waits assume whole stages in order
#pragma unroll
        for (int d = 0; d < D; ++d) issue_wq(st[d], min(g0 + d * kStep, G - 1), d < cnt);
        inputs_ready();
#pragma unroll
        for (int d = 0; d < D; ++d) issue_x(st[d], d, min(g0 + d * kStep, G - 1), d < cnt);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    else {
#pragma unroll
        for (int d = 0; d < D; ++d) issue(st[d], d, min(g0 + d * kStep, G - 1), d < cnt);
    }
    // D groups per trip, so that each stage keeps its registers; all conditions are wave-uniform
    // and none of them surrounds a load.
    for (int i = 0; i < cnt; i += D) {
        static_for<0, D>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            step(dc, i + d < cnt, g0 + (i + d + D) * kStep, i + d + D < cnt);
        });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the masked refills of the last trip

    // ---- add the eight slices in LDS, in slice order ----
    // red[slice][r][h][lane] as float4, over the activation patches: every wave must be done with its own
    __syncthreads();
    float4_t* red4 = reinterpret_cast<float4_t*>(smem);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int h = 0; h < H; ++h) red4[((wave * R + r) * H + h) * 64 + lane] = acc[h][r];
    __syncthreads();
    for (int rh = wave; rh < R * H; rh += NW) {  // (tile r, row block h) is finished by wave r * H + h (mod NW)
        const int r = rh / H, h = rh % H;
        float4_t  v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NW; ++s) v += red4[((s * R + r) * H + h) * 64 + lane];

        // ---- epilogue: lane (c, b) holds column n = 16 * (col0 + r) + c, tokens t0 + 16h + 4b + i ----
        const int n   = (col0 + r) * kTileN + c;
        const int epi = EPI == kEpiRuntime ? p.epilogue : EPI;
        auto put = [&](int64_t at, half_t o) {
            const uint16_t bits = __builtin_bit_cast(uint16_t, o);
            if constexpr (SEQ) __hip_atomic_store(p.C + at, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else p.C[at] = bits;
        };
        // (the four residual loads of a lane are issued together: at agent scope each is a trip to memory)
        uint16_t rb[4] = {0, 0, 0, 0};
        if (epi == kEpiAdd) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 16 * h + 4 * b + i;
                if (row < Tl) {
                    const int64_t at = (int64_t)(t0 + row) * N + n;
                    if constexpr (SEQ) rb[i] = __hip_atomic_load(p.Rsd + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else rb[i] = p.Rsd[at];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half_t hv    = (half_t)v[i];
            const int    row   = 16 * h + 4 * b + i;
            const int    token = t0 + row;
            if (epi == kEpiSilu) {
                // gate = even column, up = odd column: fetch the neighbour lane's value
                const float mine  = (float)hv;
                const float other = __shfl_xor(mine, 1);
                if (row < Tl && (c & 1) == 0) put((int64_t)token * (N / 2) + (n >> 1), (half_t)(mine / (1.f + __expf(-mine)) * other));
            }
            else if (row < Tl) {
                const int64_t at = (int64_t)token * N + n;
                if (epi == kEpiGemm) put(at, hv);
                else put(at, (half_t)((float)__builtin_bit_cast(half_t, rb[i]) + (float)hv));
            }
        }
    }
}

}  // namespace strip

}  // namespace w4a16
