// Prefill W4A16 GEMM for gfx950: many tokens, bound by the fp16 MFMA rate.
//
// A workgroup of four (or eight) waves computes a (16*TTILES tokens) x (16*NTW*WAVES features)
// output tile.
// The waves split the features; each owns NTW weight tiles per quantisation group and loads
// them straight from global memory into registers (one 128-bit load per lane and tile: the
// tiled layout IS the MFMA operand layout), dequantises them to the reference's exact fp16
// weight fp16_rn((q - z) * s) and uses them as the A operand of v_mfma_f32_16x16x32_f16.
// The activations of the tile go from global memory directly into LDS (no registers, no
// ds_write), D buffers deep, one 128-wide K step per quantisation group, and are read as the
// B operand by all waves, so no weight is dequantised twice and no activation is fetched
// twice per workgroup.  With weights as A the accumulator of a lane holds four adjacent
// features of one token, which makes every epilogue (plain, SiLU-gate on feature pairs,
// residual add) lane-local.
//
// The K loop is one hand-scheduled instruction stream per wave: every MFMA is followed by its
// share of the NEXT sub-step's (one or two k32 chunks) dequantisation, LDS fragment reads and
// global loads, so that a single wave keeps the matrix pipe busy while it issues everything else (measured on this
// part: an MFMA occupies the pipe for 16 cycles and issues in 4; two vector instructions fit
// behind each one for free, a third does not).  The MFMAs are inline assembly with the
// accumulators tied in place in AGPRs; loads are inline assembly waited for by count.
#include "w4a16_common.h"
#include "w4a16_internal.h"

#include <cmath>
#include <type_traits>

namespace w4a16 {

namespace {

// LDS holds two activation tiles of [tokens][128 halves] = 256 bytes per token row, i.e. 16 chunks
// of 16 bytes.  Chunk position p of row r holds K-chunk p ^ (r & 15): the 16 lanes that read the
// same K-chunk of 16 consecutive rows then hit 16 different bank groups, without padding, which
// the direct global-to-LDS loads (64 lanes x 16 contiguous bytes) could not produce.
constexpr int kRowBytes = kGroup * 2;

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(<N-1>); gives inline assembly
// its immediate operands.
template<int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Loads of the software pipeline.  They are issued from inline assembly, in place ("+v"), with
// a scalar base and a per-thread 32-bit offset, and waited for by count: the compiler would
// drain every load in flight at the loop header, exposing the memory latency once per K step.
template<int OFF>
__device__ __forceinline__ void gload128(u32x4_t& dst, uint32_t voff, const void* sbase)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF));
}
template<int OFF>
__device__ __forceinline__ void gload32(uint32_t& dst, uint32_t voff, const void* sbase)
{
    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "+v"(dst) : "v"(voff), "s"(sbase), "n"(OFF));
}
// Global memory straight into LDS: lane l's 16 bytes land at lds_base + 16 l.  The LDS base travels
// in M0; written here (rather than through the builtin) so that the address is a scalar base
// plus a 32-bit lane offset instead of a 64-bit lane address, which costs a register pair and an
// add per request.
__device__ __forceinline__ uint32_t lds_addr(const void* p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(p);
}
__device__ __forceinline__ void gload_lds128(uint32_t lds_base, uint32_t voff, const void* sbase)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_base)
                 : "memory", "m0");
}
// wait until at most N of this wave's loads are in flight; tied to `v` so that no use of it can
// be scheduled above the wait
template<int N, typename V>
__device__ __forceinline__ void wait_vm(V& v)
{
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N));
}

// LDS fragment read from inline assembly (byte address + immediate), and its wait.  Left to the
// compiler, each activation fragment was read right before the MFMAs that use it, which then
// waited a full LDS latency; and any compiler-visible LDS read after a direct-to-LDS load would
// be preceded by a wait for ALL loads in flight.  Here the fragments of a sub-step are requested
// during the previous one.
template<int OFF>
__device__ __forceinline__ void lds_read128(half8_t& dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ void wait_lgkm0(half8_t& a, half8_t& b, half8_t& c, half8_t& d)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

__device__ __forceinline__ uint64_t pack2(float a, float b)
{
    return (uint64_t)__builtin_bit_cast(uint32_t, a) | ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
}
__device__ __forceinline__ float lo_float(uint64_t v) { return __builtin_bit_cast(float, (uint32_t)v); }
__device__ __forceinline__ float hi_float(uint64_t v) { return __builtin_bit_cast(float, (uint32_t)(v >> 32)); }

// Register budget: one wave per SIMD (512 registers) for the 128-register accumulator tiles,
// two waves otherwise.  Stating it keeps the allocator from squeezing the kernel into fewer
// VGPRs and parking values in AGPRs, which is fatal here: a register parked while an
// inline-assembly load into it is still in flight is handed to another value, and the load then
// lands on that value (the build rejects kernels that use AGPRs beyond their accumulators).
// WAVES = waves per workgroup (4 or 8), side by side along the features.
// D = groups in flight per wave (2 or 4): the loads of group g + D are issued while group g is
// being multiplied.  Two cover the memory latency when a K step is long (large tiles); small tiles
// finish a step in a fraction of that and need four.
// KS = k32 chunks per sub-step (1 or 2).  The operands of a sub-step - activation fragments from
// LDS, dequantised weights - are requested and prepared during the previous one.  A 64-token tile
// has only 4 * NTW MFMAs per k32 chunk, too few to cover the LDS latency; two chunks per sub-step
// double the cover at the price of a second set of fragment registers.
// NQ = quantisation groups per 128-row weight tile: 1 (group size 128), 2 (64) or 4 (32).  A K step is still one
// weight tile; with NQ > 1 every k32 chunk (or pair of chunks) of the tile has its own scale and zero point, which
// are taken from the tile's NQ Q words right before the chunk is dequantised instead of once per K step.
template<int TTILES, int NTW, int WAVES, int D, int KS, int EPI, int NQ = 1>
__global__ void __launch_bounds__(64 * WAVES)
    __attribute__((amdgpu_waves_per_eu(TTILES * NTW * KS >= 16 && WAVES == 4 && (TTILES * NTW >= 32 || KS == 2) ? 1 : 2,
                                       TTILES * NTW * KS >= 16 && WAVES == 4 && (TTILES * NTW >= 32 || KS == 2) ? 1 : 2)))
prefill_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
               const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K, int tiles_t, int tiles_n,
               float* ws, int* cnt)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];  // [D][TT][kRowBytes]
    constexpr int TT = 16 * TTILES;
    constexpr int TN = 16 * NTW * WAVES;
    constexpr int XB = 4 * TTILES / WAVES;  // 1 KiB activation blocks (4 token rows) that each wave fetches per group
    static_assert(4 * TTILES % WAVES == 0, "the activation tile must divide evenly among the waves");
    static_assert(D == 2 || D == 4, "stages alternate in parity, so their number is even");
    static_assert(KS == 1 || KS == 2, "a group is four k32 chunks; sub-steps alternate in parity");
    constexpr int kSub = 4 / KS;  // sub-steps per group

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c    = lane & 15;
    const int b    = lane >> 4;
    const int G    = K / kGroup;
    const int NT   = N / kTileN;

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles so
    // its private L2 sees the reuse.  Inside a run, tiles go four token tiles at a time across
    // the feature tiles: the ~64 workgroups an XCD runs concurrently then cover 4 token tiles x
    // 16 feature tiles, which minimises what they fetch together (a token tile of activations
    // is four times larger than a feature tile of int4 weights).
    const int total = tiles_t * tiles_n;
    int       id    = blockIdx.x;
    if (total % 8 == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    int tile_t, tile_n;
    if (tiles_t % 4 == 0) {
        const int r = id >> 2;
        tile_n      = r % tiles_n;
        tile_t      = (r / tiles_n) * 4 + (id & 3);
    }
    else {
        tile_t = id % tiles_t;
        tile_n = id / tiles_t;
    }
    // split K: blockIdx.y takes the quantisation groups [gbeg, gend), dealt in pairs so that only
    // the last split can have an odd number of them
    const int splits = gridDim.y;
    const int pairs  = (G + 1) / 2;
    const int gbeg   = min(G, 2 * (int)((int64_t)pairs * blockIdx.y / splits));
    const int gend   = min(G, 2 * (int)((int64_t)pairs * (blockIdx.y + 1) / splits));
    const int T0     = tile_t * TT;
    const int nt0    = (tile_n * TN) / kTileN + wave * NTW;  // first weight tile of this wave

    // per-thread byte offsets; the group-dependent part of every address is scalar
    const uint32_t w_off = (uint32_t)(nt0 * 1024 + lane * 16);        // + g * NT * 1024 (+ nt * 1024)
    const uint32_t q_off = (uint32_t)((nt0 * kTileN + c) * 4);        // + g * N * 4    (+ nt * 64)
    // X staging, direct global -> LDS: wave w, request i writes the 1 KiB block m = w*XB + i
    // (token rows 4m .. 4m+3) of the tile; lane l lands at row 4m + l/16, chunk position l%16, so it
    // fetches K-chunk (l%16) ^ (row & 15) of that row.  Rows past the last token re-read the last
    // valid row; their outputs are never stored.
    uint32_t x_off[XB];
#pragma unroll
    for (int i = 0; i < XB; ++i) {
        const int row = 4 * (wave * XB + i) + (lane >> 4);
        x_off[i] = (uint32_t)min(T0 + row, T - 1) * (uint32_t)(K * 2) + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
    }
    // fragment reads: lane (c, b) reads row 16*tt + c, K-chunk 4j + b  ->  position (4j + b) ^ c
    uint32_t xr_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) xr_off[j] = (uint32_t)(c * kRowBytes + (((4 * j + b) ^ c) & 15) * 16);

    const UnpackConsts uc;

    float4_t acc[TTILES][NTW];
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) acc[tt][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

    static_assert(NQ == 1 || NQ == 2 || NQ == 4, "group sizes 128, 64 and 32");
    constexpr int NQW = NTW * NQ;  // Q words per K step: tile nt's are qv[nt * NQ ..]
    u32x4_t  w[D][NTW];  // weights and (scale, zero) words of the D groups in flight; stage = group index mod D
    uint32_t q[D][NQW];
#pragma unroll
    for (int d = 0; d < D; ++d) {
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) w[d][nt] = u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < NQW; ++i) q[d][i] = 0;
    }

    auto issue_w = [&](u32x4_t (&ws_)[NTW], uint32_t (&qv)[NQW], int g) {
        const char* wbase = reinterpret_cast<const char*>(A) + (int64_t)g * NT * 1024;
        const char* qbase = reinterpret_cast<const char*>(Q) + (int64_t)g * NQ * N * 4;
        static_for<0, NTW>([&](auto nt) { gload128<nt * 1024>(ws_[nt], w_off, wbase); });
        static_for<0, NQW>([&](auto i) {
            constexpr int nt = decltype(i)::value / NQ, sub = decltype(i)::value % NQ;
            gload32<nt * 64>(qv[decltype(i)::value], q_off, qbase + (int64_t)sub * N * 4);
        });
    };
    // the activation tile of group g, straight into the LDS buffer `xo` (no registers, no ds_write)
    auto issue_x = [&](uint8_t* xo, int g) {
        const char* xbase = reinterpret_cast<const char*>(X) + (int64_t)g * 256;
#pragma unroll
        for (int i = 0; i < XB; ++i) gload_lds128(lds_addr(xo) + (wave * XB + i) * 1024, x_off[i], xbase);
    };
    // the same requests one at a time (m = 0 .. 2 NTW + TTILES - 1), to be dealt out between MFMAs
    constexpr int kVmOps = NTW + NQW + XB;
    auto vm_op = [&](auto M, u32x4_t (&ws_)[NTW], uint32_t (&qv)[NQW], uint8_t* xo, const char* wbase, const char* qbase,
                     const char* xbase) {
        constexpr int m = decltype(M)::value;
        if constexpr (m < NTW) {
            gload128<m * 1024>(ws_[m], w_off, wbase);
        }
        else if constexpr (m < NTW + NQW) {
            constexpr int nt = (m - NTW) / NQ, sub = (m - NTW) % NQ;
            gload32<nt * 64>(qv[m - NTW], q_off, qbase + (int64_t)sub * N * 4);
        }
        else {
            constexpr int i = m - NTW - NQW;
            gload_lds128(lds_addr(xo) + (wave * XB + i) * 1024, x_off[i], xbase);
        }
    };
    // wait until at most `Pending` younger stages' loads are in flight, then release the stage's registers
    auto wait_stage = [&](auto Pending, u32x4_t (&ws_)[NTW], uint32_t (&qv)[NQW]) {
        constexpr int n = decltype(Pending)::value * kVmOps;
        static_assert(n <= 63, "vmcnt is a 6-bit counter");
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) wait_vm<n>(ws_[nt]);
#pragma unroll
        for (int i = 0; i < NQW; ++i) wait_vm<n>(qv[i]);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // State carried from one sub-step to the next (and across K steps): dequantised weights and
    // activation fragments of the current / next sub-step, zero points and scale of the current /
    // next group.
    half8_t wf[2][KS][NTW];   // [sub-step parity][chunk][tile]
    half8_t xf[2][KS][TTILES];
    half2_t z1024[2][NTW], z64[2][NTW], sc[2][NTW];

    auto split = [&](auto P_, uint32_t (&qv)[NQW]) {
        constexpr int P = decltype(P_)::value;
        if constexpr (NQ > 1) return;  // (taken chunk by chunk inside dequant_op)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) {
            half_t s;
            split_q(qv[nt], z1024[P][nt], z64[P][nt], s);
            sc[P][nt] = half2_t{s, s};
        }
    };
    // The dequantisation of word J of every tile of `w`, as 13 * NTW single vector instructions
    // (op = NTW * k + nt) so that they can be dealt out between the MFMAs of a sub-step:
    // k = 0: w >> 8;  1..4: (w & mask) | magic;  5..8: - (offset + zero);  9..12: * scale.
    uint32_t dq[NTW][5];
    auto dequant_op = [&](auto P, auto J, auto OP, u32x4_t (&ws_)[NTW], uint32_t (&qv)[NQW]) {
        // (NQ > 1: the zero points and the scale of word j's quantisation group replace parity p's for this word)
        constexpr int p = NQ > 1 ? 0 : decltype(P)::value, j = decltype(J)::value;
        constexpr int nt = decltype(OP)::value % NTW, k = decltype(OP)::value / NTW;
        if constexpr (k == 0 && NQ > 1) {
            half_t s;
            split_q(qv[nt * NQ + j * NQ / 4], z1024[0][nt], z64[0][nt], s);
            sc[0][nt] = half2_t{s, s};
        }
        if constexpr (k == 0) dq[nt][4] = ws_[nt][j] >> 8;
        else if constexpr (k <= 4) {
            constexpr int i  = k - 1;
            const uint32_t src = i < 2 ? ws_[nt][j] : dq[nt][4];
            dq[nt][i] = (src & (i & 1 ? uc.mask_hi : uc.mask_lo)) | (i & 1 ? uc.magic_hi : uc.magic_lo);
        }
        else if constexpr (k <= 8) {
            constexpr int i = k - 5;
            dq[nt][i]       = as_u32(as_half2(dq[nt][i]) - (i & 1 ? z64[p][nt] : z1024[p][nt]));
        }
        else {
            constexpr int i = k - 9;
            const half2_t r = as_half2(dq[nt][i]) * sc[p][nt];
            wf[(j / KS) & 1][j % KS][nt][2 * i]     = r[0];
            wf[(j / KS) & 1][j % KS][nt][2 * i + 1] = r[1];
        }
    };
    auto dequant = [&](auto P, auto J, u32x4_t (&ws_)[NTW], uint32_t (&qv)[NQW]) {
        static_for<0, 13 * NTW>([&](auto op) { dequant_op(P, J, op, ws_, qv); });
    };
    auto read_x = [&](auto J_, const uint8_t* xb) {
        constexpr int  J    = decltype(J_)::value;
        const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(xb) + xr_off[J];
        static_for<0, TTILES>([&](auto tt) { lds_read128<tt * 16 * kRowBytes>(xf[(J / KS) & 1][J % KS][tt], addr); });
    };
    auto read_x1 = [&](auto J_, auto TT_, uint32_t base) {
        constexpr int J = decltype(J_)::value, tt = decltype(TT_)::value;
        lds_read128<tt * 16 * kRowBytes>(xf[(J / KS) & 1][J % KS][tt], base + xr_off[J]);
    };
    // ---- prologue: the first D groups in flight, first operands of the first one prepared ----
    // The K loop works through the groups D at a time (the D parts of its body differ in which
    // registers and which LDS buffer hold the current group).  A group count that is not a
    // multiple of D is padded with phantom groups in front: their activation tile is zero-filled
    // LDS instead of a load and their weights are those of the first real group, so they add
    // exactly zero.
    const int pad    = (D - (gend - gbeg) % D) % D;
    const int gstart = gbeg - pad;
    static_for<0, D>([&](auto dc) {
        constexpr int d  = decltype(dc)::value;
        uint8_t* const xd = xs + d * TT * kRowBytes;
        issue_w(w[d], q[d], max(gstart + d, gbeg));
        if (gstart + d < gbeg) {
            for (int i = tid; i < TT * 16; i += 64 * WAVES) reinterpret_cast<u32x4_t*>(xd)[i] = u32x4_t{0, 0, 0, 0};
        }
        else {
            issue_x(xd, gstart + d);
        }
    });
    static_for<0, D>([&](auto dc) { wait_stage(I0{}, w[decltype(dc)::value], q[decltype(dc)::value]); });
    __syncthreads();
    split(I0{}, q[0]);
    static_for<0, KS>([&](auto kc) {
        read_x(kc, xs);
        dequant(I0{}, kc, w[0], q[0]);
    });

    // One K step (a quantisation group, four k32 chunks in kSub sub-steps) on stage S: weights w[S],
    // LDS buffer S, group parity S & 1.  Every sub-step runs its MFMAs interleaved with the
    // dequantisation of the NEXT sub-step's weights and the requests for its activation fragments.
    // In the last sub-step the next group's weights (stage S + 1, requested D - 1 K steps ago) and
    // activation tile are complete: the workgroup synchronises, starts on them, and re-uses stage
    // S, which no wave reads any more, for the loads of group g + D.
    auto step = [&](auto S_, int g) {
        constexpr int S = decltype(S_)::value, SN = (S + 1) % D;
        constexpr int p = S & 1;
        using P          = std::integral_constant<int, p>;
        using PN         = std::integral_constant<int, p ^ 1>;
        uint8_t* const       xb = xs + S * TT * kRowBytes;
        const uint8_t* const xo = xs + SN * TT * kRowBytes;
        static_for<0, kSub>([&](auto sc_) {
            constexpr int  sub  = decltype(sc_)::value;
            constexpr bool last = sub == kSub - 1;
            constexpr int  par  = sub & 1;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk)
#pragma unroll
                for (int tt = 0; tt < TTILES; tt += 4)
                    wait_lgkm0(xf[par][kk][tt], xf[par][kk][tt + 1], xf[par][kk][tt + 2], xf[par][kk][tt + 3]);
            const int   g2 = min(g + D, gend - 1);  // (the last steps re-read the last group: no branch)
            const char* wbase = reinterpret_cast<const char*>(A) + (int64_t)g2 * NT * 1024;
            const char* qbase = reinterpret_cast<const char*>(Q) + (int64_t)g2 * NQ * N * 4;
            const char* xbase = reinterpret_cast<const char*>(X) + (int64_t)g2 * 256;
            if constexpr (last) {
                // stages S + 2 .. S + D - 1 may still be in flight behind stage S + 1
                wait_stage(std::integral_constant<int, D - 2>{}, w[SN], q[SN]);
                __syncthreads();
            }
            const uint32_t rbase =
                (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)(last ? xo : (const uint8_t*)xb);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (last) split(PN{}, q[SN]);
            // one MFMA, then its share of the next sub-step's dequantisation, and so on
            constexpr int kOps = 13 * NTW * KS, kSlots = TTILES * NTW * KS, kReads = TTILES * KS;
            static_for<0, kSlots>([&](auto ic) {
                constexpr int i = decltype(ic)::value, kk = i / (TTILES * NTW), tt = i % (TTILES * NTW) / NTW, nt = i % NTW;
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                             : "+a"(acc[tt][nt])
                             : "v"(wf[par][kk][nt]), "v"(xf[par][kk][tt]));
                __builtin_amdgcn_sched_barrier(0);
                // (word = chunk of the next sub-step, 13 * NTW operations each, in order: they share temporaries)
                static_for<i * kOps / kSlots, (i + 1) * kOps / kSlots>([&](auto op) {
                    constexpr int word = decltype(op)::value / (13 * NTW);
                    using OP           = std::integral_constant<int, decltype(op)::value % (13 * NTW)>;
                    if constexpr (!last) dequant_op(P{}, std::integral_constant<int, (sub + 1) * KS + word>{}, OP{}, w[S], q[S]);
                    else dequant_op(PN{}, std::integral_constant<int, word>{}, OP{}, w[SN], q[SN]);
                });
                // the next sub-step's activation fragments, requested during the first three quarters
                // of this one; in the last sub-step also the loads of group g + D
                constexpr int kR = kSlots * 3 / 4 > 0 ? kSlots * 3 / 4 : 1;
                if constexpr (i < kR) {
                    static_for<i * kReads / kR, (i + 1) * kReads / kR>([&](auto rd) {
                        constexpr int chunk = (last ? 0 : (sub + 1) * KS) + decltype(rd)::value / TTILES;
                        read_x1(std::integral_constant<int, chunk>{},
                                std::integral_constant<int, decltype(rd)::value % TTILES>{}, rbase);
                    });
                }
                if constexpr (last) {
                    static_for<i * kVmOps / kSlots, (i + 1) * kVmOps / kSlots>(
                        [&](auto m) { vm_op(m, w[S], q[S], xb, wbase, qbase, xbase); });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };

    // Whole multiples of D only (see `pad` above): no K step outside the loop, so the compiler never
    // has a reason to move an accumulator while the loop's MFMAs may still be writing it.
    for (int g = gstart; g + D - 1 < gend; g += D) {  // no branch inside: the 4*TTILES*NTW accumulators stay in place
        static_for<0, D>([&](auto dc) { step(dc, g + decltype(dc)::value); });
    }
    // no load may still be writing LDS or registers when the wave ends
    static_for<0, D>([&](auto dc) { wait_stage(I0{}, w[decltype(dc)::value], q[decltype(dc)::value]); });
    // The last sub-step requested activation fragments for a step that does not exist.  Nothing
    // reads them, so the compiler may hand their registers out again at once while the LDS reads
    // are still on their way and would land on the new owner: wait for them first.  (Tying the
    // registers to the wait would keep both fragment sets alive and cost registers in the loop;
    // the build's assembly check verifies instead that nothing touches them before this wait.)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // the MFMAs are inline assembly, so the compiler does not know that the accumulators are
    // still being written: cover the longest MFMA-result-to-VALU-read distance by hand (the
    // build's assembly check verifies that no accumulator is read before this)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // the epilogue of one 16 x 16 tile: lane (c, b) holds token T0 + 16 tt + c, features n .. n+3
    auto emit = [&](int tt, int nt, const float4_t v) {
        const int token = T0 + tt * 16 + c;
        if (token >= T) return;
        const int    n  = (nt0 + nt) * kTileN + 4 * b;
        const half_t h0 = (half_t)v[0], h1 = (half_t)v[1], h2 = (half_t)v[2], h3 = (half_t)v[3];
        if constexpr (EPI == kEpiGemm) {
            uint2 o;
            o.x = as_u32(half2_t{h0, h1});
            o.y = as_u32(half2_t{h2, h3});
            *reinterpret_cast<uint2*>(C + (int64_t)token * N + n) = o;
        }
        else if constexpr (EPI == kEpiSilu) {
            const float  g0 = (float)h0, u0 = (float)h1, g1 = (float)h2, u1 = (float)h3;
            const half_t o0 = (half_t)(g0 / (1.f + __expf(-g0)) * u0);
            const half_t o1 = (half_t)(g1 / (1.f + __expf(-g1)) * u1);
            *reinterpret_cast<uint32_t*>(C + (int64_t)token * (N / 2) + (n >> 1)) = as_u32(half2_t{o0, o1});
        }
        else {
            const uint2   rr = *reinterpret_cast<const uint2*>(R_ + (int64_t)token * N + n);
            const half2_t r0 = as_half2(rr.x), r1 = as_half2(rr.y);
            uint2         o;
            o.x = as_u32(half2_t{(half_t)((float)r0[0] + (float)h0), (half_t)((float)r0[1] + (float)h1)});
            o.y = as_u32(half2_t{(half_t)((float)r1[0] + (float)h2), (half_t)((float)r1[1] + (float)h3)});
            *reinterpret_cast<uint2*>(C + (int64_t)token * N + n) = o;
        }
    };

    // ---- split K: exchange partial tiles through the workspace ----
    // Each wave writes its accumulators as it holds them (per tile two 512-byte rows, lane l the
    // floats 2l, 2l+1), with agent-scope atomic stores and loads: the L2 caches of the XCDs are not
    // coherent with each other, and these go through to memory without a full cache write-back.
    // A store is complete when the wave's store counter drains, so draining it before the arrival
    // counter is incremented orders the two.  The last workgroup to arrive adds the partial tiles
    // in split order, its own included, so the sum does not depend on which one is last.
    if (splits > 1) {
        constexpr int kTiles = TTILES * NTW;
        const int64_t per_split = (int64_t)total * WAVES * kTiles * 256;  // floats
        // (the lane index is hidden from the optimiser here so that none of these addresses is
        // computed before the K loop and carried through it in registers)
        int lane_now = lane;
        asm volatile("" : "+v"(lane_now));
        float* const  mine_base = ws + ((int64_t)id * WAVES + wave) * kTiles * 256 + lane_now * 2;
        {
            float* wp = mine_base + blockIdx.y * per_split;
#pragma unroll
            for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
                for (int nt = 0; nt < NTW; ++nt) {
                    const float4_t v = acc[tt][nt];
                    uint64_t*      o = reinterpret_cast<uint64_t*>(wp + (tt * NTW + nt) * 256);
                    __hip_atomic_store(o, pack2(v[0], v[1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(o + 64, pack2(v[2], v[3]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        }
        __builtin_amdgcn_s_waitcnt(0);  // all of this wave's stores are complete
        __syncthreads();                // ... and every wave is done with the activation tiles in LDS
        int* const last_flag = reinterpret_cast<int*>(xs);
        if (tid == 0) {
            int* const cp   = cnt + id;
            const int  old  = __hip_atomic_fetch_add(cp, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool last = old == splits - 1;
            if (last) __hip_atomic_store(cp, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
            *last_flag = last;
        }
        __syncthreads();
        if (!*last_flag) return;
#pragma unroll
        for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
            for (int nt = 0; nt < NTW; ++nt) {
                float4_t sum = {0.f, 0.f, 0.f, 0.f};
                // four splits' loads in flight at a time
                for (int s0 = 0; s0 < splits; s0 += 4) {
                    uint64_t v[4][2];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const uint64_t* ip = reinterpret_cast<const uint64_t*>(
                            mine_base + min(s0 + u, splits - 1) * per_split + (tt * NTW + nt) * 256);
                        v[u][0] = __hip_atomic_load(ip, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        v[u][1] = __hip_atomic_load(ip + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (s0 + u < splits) {
                            sum[0] += lo_float(v[u][0]); sum[1] += hi_float(v[u][0]);
                            sum[2] += lo_float(v[u][1]); sum[3] += hi_float(v[u][1]);
                        }
                    }
                }
                emit(tt, nt, sum);
            }
        return;
    }

    // ---- epilogue: lane (c, b) of tile (tt, nt) holds token T0 + 16 tt + c, features n .. n+3 ----
#pragma unroll
    for (int tt = 0; tt < TTILES; ++tt)
#pragma unroll
        for (int nt = 0; nt < NTW; ++nt) emit(tt, nt, acc[tt][nt]);
}

struct Variant {
    int ttiles, ntw, waves, depth, chunks;
    // Measured on MI355X (K = 2048 against 6144, cold weights): microseconds per K step for the whole
    // grid at 1, 2, 3, 4 and 8 workgroups per CU.  Tiles that fill a CU by themselves go in rounds.
    // (The two-chunk rows are the one-chunk measurements x 0.96, the ratio seen on Llama-7B shapes.)
    bool  one_per_cu;
    float step_us[5];
};
// (a 256 x 256 tile does not fit the register file without spilling, and spill stores would
// break the counted waits: stores and loads complete out of order with each other)
constexpr Variant kVariants[] = {
    {8, 2, 8, 2, 1, true, {1.810f, 3.630f, 5.240f, 6.740f, 12.980f}},   // 128 x 256, eight waves
    {16, 2, 4, 2, 1, true, {2.071f, 4.498f, 6.126f, 8.397f, 15.010f}},  // 256 x 128
    {8, 2, 4, 2, 1, false, {1.016f, 1.860f, 3.067f, 4.002f, 7.185f}},   // 128 x 128
    {4, 2, 4, 4, 1, false, {0.672f, 1.111f, 1.664f, 2.271f, 4.773f}},   //  64 x 128
    {4, 1, 4, 4, 2, false, {0.425f, 0.673f, 1.000f, 1.340f, 2.833f}},   //  64 x 64, two chunks per sub-step
    {4, 1, 8, 4, 2, true, {0.553f, 1.209f, 1.906f, 2.609f, 5.351f}},    //  64 x 128, eight waves, two chunks per sub-step
    {4, 2, 8, 4, 1, true, {1.034f, 2.290f, 3.605f, 4.644f, 8.583f}},    //  64 x 256, eight waves
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template<int TTILES, int NTW, int WAVES, int D, int KS, int NQ = 1>
hipError_t launch_v(int splits, const GemmArgs& a, const Scratch& sc, hipStream_t st)
{
    constexpr int TT = 16 * TTILES, TN = 16 * NTW * WAVES;
    const int     tiles_t = (a.T + TT - 1) / TT;
    const int     tiles_n = a.N / TN;
    const size_t  lds     = (size_t)D * TT * kRowBytes;
    const dim3    grid(tiles_t * tiles_n, splits), block(64 * WAVES);
    const u32x4_t* A4 = reinterpret_cast<const u32x4_t*>(a.A);
#define W4A16_LAUNCH(EPI)                                                                                              \
    do {                                                                                                               \
        auto                         kfn = prefill_kernel<TTILES, NTW, WAVES, D, KS, EPI, NQ>;                         \
        static std::atomic<uint64_t> raised{0}; /* per instantiation, one bit per device */                            \
        const hipError_t             e = raise_lds_limit(reinterpret_cast<const void*>(kfn), (int)lds, raised);        \
        if (e != hipSuccess) return e;                                                                                 \
        return launch_kernel(kfn, grid, block, lds, st, a.C, A4, a.X, a.Q, a.R, a.N, a.T, a.K, tiles_t, tiles_n,       \
                             sc.ws, sc.cnt);                                                                           \
    } while (0)
    switch (a.epilogue) {
        case kEpiGemm: W4A16_LAUNCH(kEpiGemm);
        case kEpiSilu: W4A16_LAUNCH(kEpiSilu);
        default: W4A16_LAUNCH(kEpiAdd);
    }
#undef W4A16_LAUNCH
}

}  // namespace

int prefill_variants()
{
    return kNumVariants;
}

void prefill_tile(int v, int& tile_n, int& tile_t)
{
    tile_n = 16 * kVariants[v].ntw * kVariants[v].waves;
    tile_t = 16 * kVariants[v].ttiles;
}

size_t prefill_scratch_bytes(int v, int splits, int N, int T, int K)
{
    (void)K;
    if (v < 0 || v >= kNumVariants || splits <= 1) return 0;
    const int tn = 16 * kVariants[v].ntw * kVariants[v].waves, tt = 16 * kVariants[v].ttiles;
    return (size_t)(N / tn) * ((T + tt - 1) / tt) * splits * tn * tt * 4;
}

bool prefill_feasible(int v, int splits, int N, int T, int K, size_t ws_bytes, int cnt_len)
{
    if (v < 0 || v >= kNumVariants || N <= 0 || T <= 0 || K <= 0 || splits < 1) return false;
    const int tn = 16 * kVariants[v].ntw * kVariants[v].waves, tt = 16 * kVariants[v].ttiles;
    if (N % tn != 0 || K % kGroup != 0) return false;
    // per-thread offsets into X and into one group of A are 32-bit
    if ((int64_t)T * K * 2 >= (1ll << 32) || (int64_t)N * 64 >= (1ll << 32)) return false;
    const int64_t grid = (int64_t)(N / tn) * ((T + tt - 1) / tt);
    if (splits > 1) {
        // at least two groups per split; partial tiles and counters must fit the handle's scratch
        if (K / kGroup < 2 * splits || splits > 65535) return false;
        if (grid * splits * tn * tt * 4 > (int64_t)ws_bytes || grid > cnt_len) return false;
    }
    return grid * splits < (1ll << 31);
}

int prefill_grid(int v, int splits, int N, int T, int K)
{
    (void)K;
    const int tn = 16 * kVariants[v].ntw * kVariants[v].waves, tt = 16 * kVariants[v].ttiles;
    return (N / tn) * ((T + tt - 1) / tt) * splits;
}

hipError_t prefill_launch(int v, int splits, const GemmArgs& a, const Scratch& sc, hipStream_t st)
{
    if (splits > 1 && (sc.ws == nullptr || sc.cnt == nullptr)) return hipErrorInvalidValue;
    switch (v) {
        case 0: return launch_v<8, 2, 8, 2, 1>(splits, a, sc, st);
        case 1: return launch_v<16, 2, 4, 2, 1>(splits, a, sc, st);
        case 2: return launch_v<8, 2, 4, 2, 1>(splits, a, sc, st);
        case 3: return launch_v<4, 2, 4, 4, 1>(splits, a, sc, st);
        case 4: return launch_v<4, 1, 4, 4, 2>(splits, a, sc, st);
        case 5: return launch_v<4, 1, 8, 4, 2>(splits, a, sc, st);
        default: return launch_v<4, 2, 8, 4, 1>(splits, a, sc, st);
    }
}

// Group sizes 64 and 32 (nq = 2, 4): the 256-token x 128-feature tile, the one variant with registers to spare for
// the extra Q words of a K step.
bool prefill_groups_feasible(int nq, int N, int T, int K)
{
    return (nq == 2 || nq == 4) && prefill_feasible(1, 1, N, T, K, 0, 0);
}

hipError_t prefill_groups_launch(int nq, const GemmArgs& a, hipStream_t st)
{
    if (!prefill_groups_feasible(nq, a.N, a.T, a.K)) return hipErrorInvalidValue;
    const Scratch none{};
    return nq == 2 ? launch_v<16, 2, 4, 2, 1, 2>(1, a, none, st) : launch_v<16, 2, 4, 2, 1, 4>(1, a, none, st);
}

// Predicted run time in microseconds, from the measured step times: launch and epilogue, the K
// steps of one workgroup at the load the grid puts on the chip, and for split K the exchange of
// partial tiles.
double prefill_estimate_us(int v, int splits, int N, int T, int K)
{
    const Variant& var = kVariants[v];
    const int      tn = 16 * var.ntw * var.waves, tt = 16 * var.ttiles;
    const double   wgs  = (double)(N / tn) * ((T + tt - 1) / tt) * splits;
    const double   load = wgs / 256.0;
    // tiles that fill a CU by themselves go in whole rounds
    const double le = var.one_per_cu ? std::ceil(load) : load;
    double       step;
    if (le <= 4.0) {
        step = var.step_us[le <= 1.0 ? 0 : le <= 2.0 ? 1 : le <= 3.0 ? 2 : 3];
    }
    else if (le <= 8.0) {
        step = var.step_us[3] + (var.step_us[4] - var.step_us[3]) * (le - 4.0) / 4.0;
    }
    else {
        step = var.step_us[4] * le / 8.0;
    }
    // corrections from real Llama shapes: a partly idle chip clocks higher and shares less memory
    // bandwidth; 64-token tiles under heavy load ran slower than on the calibration grid
    if (var.one_per_cu && load < 1.0) step *= 0.7 + 0.3 * load;
    if (!var.one_per_cu && var.ttiles == 4 && load > 2.0) step *= 1.25;
    const int groups = K / kGroup;
    int       steps  = (groups + splits - 1) / splits;
    steps            = (steps + var.depth - 1) / var.depth * var.depth;  // phantom groups
    double us = 3.0 + steps * step;
    if (splits > 1) {
        const double tokens = (double)((T + tt - 1) / tt) * tt;
        // drain of the partial stores, arrival counter, then the last workgroup reads every split's tile
        us += 2.0 + 0.6 * splits + splits * tokens * N * 8.0 / 4.0e6;
    }
    return us;
}

}  // namespace w4a16
