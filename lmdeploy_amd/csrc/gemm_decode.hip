// Decode (skinny) W4A16 GEMM for gfx950: 16 tokens per workgroup row, bound by HBM.
//
// Work decomposition.  The weight matrix is a grid of 1 KiB tiles (16 columns x one
// 128-row quantisation group).  A workgroup has Sk "slices" of Wn waves.  It owns Wn*R
// adjacent column tiles and a range of groups; slice s takes a contiguous part of that range
// and, inside a slice, wave w streams its R column tiles with one 128-bit load per lane and
// tile, kDepth groups ahead.  The activations a slice needs are staged in LDS once per
// workgroup, already in MFMA operand order, and shared by the slice's Wn waves: the vector
// memory pipe, which moves 64 B per clock and CU whatever the access pattern, then carries
// almost only weight bytes.  Slice partial sums are added in LDS in slice order.
//
// Per group and column tile a wave computes accg[t, n] = sum_k X[t, k] * (q[k, n] - z[n])
// with v_mfma_f32_16x16x32_f16 (activations = A operand), then acc += s[n] * accg in fp32.
// The B operand of four MFMAs is the unpacked int4 still carrying its fp16 offset (1024 + q
// or 64 + q: 5 VALU instructions per 8 weights); four more MFMAs on a B operand that is
// -(offset + z) everywhere take the offsets and the zero point out again.  Every product is
// exact in fp32 and the matrix pipe is idle most of the time anyway, whereas the vector ALU is
// what bounds this kernel on large matrices.  Scaling after the group sum keeps the per-weight
// multiply out of the inner loop.  The result differs from "round every weight to fp16
// first" by that rounding (<= 2^-11 relative per term) and by the fp32 rounding of sums that
// carry the offsets (<= 2^-24 * 1039 * sum|x| per group, before scaling).
//
// Split K across workgroups (SK > 1, used only when a matrix has too few column tiles to
// fill the chip otherwise): every workgroup writes its fp32 partial tiles to a workspace,
// bumps a per-column-block counter, and the workgroup that arrives last sums the SK partials
// in split order (so the result does not depend on arrival order), applies the epilogue and
// resets the counter.  The workspace belongs to the handle; launches that share it must be
// ordered on one stream.
#include "w4a16_common.h"
#include "w4a16_internal.h"

#include <algorithm>

namespace w4a16 {

namespace {

constexpr int    kMaxWaves = 16;
constexpr size_t kMaxLds   = 128 * 1024;  // of the CU's 160 KiB; more than 64 KiB needs an opt-in per kernel

template<int R>
struct Stage {
    u32x4_t  w[R];
    uint32_t q[R];
};

struct DecodeParams {
    uint16_t*       C;
    const u32x4_t*  A;
    const uint16_t* X;
    const uint32_t* Q;
    const uint16_t* Rsd;
    float*          ws;    // [Z][SK][NT][4][64] partial accumulators
    int*            cnt;   // [Z][NB] arrival counters, zero between launches
    int             N, T, K;
    int             Wn;    // waves per slice (a power of two)
    int             lgWn;  // log2(Wn)
    int             Sk;    // slices per workgroup
    int             SK;    // K splits across workgroups
    int             GC;    // groups per slice and LDS chunk: kDepth times a power of two
    int             lgGC;  // log2(GC)
    int             per_split;  // groups per workgroup range = ceil(G / SK)
    int             per_slice;  // groups per slice = ceil(per_split / Sk)
};

// R = column tiles per wave, TP = token rows kept per activation fragment (4, 8 or 16; rows
// >= TP of the MFMA A operand repeat a lower row, which only feeds output rows that are never
// stored), kDepth = groups of weights in flight per wave.
template<int R, int TP, int kDepth, int EPI>
__global__ void __launch_bounds__(64 * kMaxWaves)
decode_kernel(const DecodeParams p)
{
    constexpr int kSlots = 16 * TP;  // 16-byte slots per group: [j][b][c]

    extern __shared__ __attribute__((aligned(16))) u32x4_t xs[];  // [Sk][GC][4][4][TP]
    __shared__ int last_flag;

    const int tid   = threadIdx.x;
    const int lane  = tid & 63;
    const int wave  = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps the loop control scalar
    const int Wn    = p.Wn;
    const int slice = wave >> p.lgWn;
    const int wn    = wave & (Wn - 1);
    const int c     = lane & 15;
    const int b     = lane >> 4;
    const int N = p.N, T = p.T, K = p.K;
    const int G  = K / kGroup;
    const int NT = N / kTileN;
    const int t0 = blockIdx.z * 16;
    const int Tl = min(16, T - t0);  // valid token rows of this workgroup

    // group range of the workgroup, then of the slice
    // (equal-length ranges, the last one shorter or empty: no division in the kernel)
    const int split = blockIdx.y;
    const int G0    = min(split * p.per_split, G);
    const int G1    = min(G0 + p.per_split, G);
    const int most  = p.per_slice;  // the longest slice: same trip count for all waves
    const int gs0   = min(G0 + slice * most, G1);
    const int gs1   = min(gs0 + most, G1);

    // column tiles of this wave; tiles past the edge are clamped for loading and not stored
    const int       nt_first = (blockIdx.x * Wn + wn) * R;
    const u32x4_t*  Ap[R];
    const uint32_t* Qp[R];
    int             nt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        nt[r] = min(nt_first + r, NT - 1);
        Ap[r] = p.A + (int64_t)nt[r] * 64 + lane;  // + g * NT * 64
        Qp[r] = p.Q + nt[r] * kTileN + c;
    }

    const UnpackConsts uc;
    const int64_t      gstride = (int64_t)NT * 64;  // 16-byte units between the tiles of consecutive groups

    auto load = [&](Stage<R>& s, int g) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            s.w[r] = __builtin_nontemporal_load(Ap[r] + g * gstride);
            s.q[r] = Qp[r][(int64_t)g * N];
        }
    };

    // Refill of a stage in the steady-state loop.  The compiler drains every load in flight at
    // a loop header (it does not count loads across the back edge), which would expose the full
    // HBM latency once per round.  These loads are therefore issued from inline assembly, in
    // place ("+v": same registers as the value they replace), and `wait_stage` below waits by
    // count for exactly the loads of the stage about to be used.
    auto refill = [&](Stage<R>& s, int g) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const u32x4_t*  wp = Ap[r] + g * gstride;
            const uint32_t* qp = Qp[r] + (int64_t)g * N;
            asm volatile("global_load_dwordx4 %0, %1, off nt" : "+v"(s.w[r]) : "v"(wp));
            asm volatile("global_load_dword %0, %1, off" : "+v"(s.q[r]) : "v"(qp));
        }
    };
    // wait until at most (kDepth - 1) stages' worth of refills are still in flight: loads return
    // in order, so the oldest stage is then complete.  Tied to the stage's registers so that no
    // use can be scheduled above the wait.
    auto wait_stage = [&](Stage<R>& s) {
        if constexpr (R == 1) {
            asm volatile("s_waitcnt vmcnt(%2)" : "+v"(s.w[0]), "+v"(s.q[0]) : "n"((kDepth - 1) * 2));
        }
        else {
            asm volatile("s_waitcnt vmcnt(%4)"
                         : "+v"(s.w[0]), "+v"(s.q[0]), "+v"(s.w[1]), "+v"(s.q[1])
                         : "n"((kDepth - 1) * 4));
        }
    };
    auto wait_all = [&](Stage<R>& s) {
        if constexpr (R == 1) {
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(s.w[0]), "+v"(s.q[0]));
        }
        else {
            asm volatile("s_waitcnt vmcnt(0)" : "+v"(s.w[0]), "+v"(s.q[0]), "+v"(s.w[1]), "+v"(s.q[1]));
        }
    };

    float4_t acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};

    // this lane's A operand inside a staged group: slot [j][b][c & (TP-1)]
    const u32x4_t* xs_me = xs + (slice * p.GC) * kSlots + b * TP + (c & (TP - 1));

    auto compute = [&](const Stage<R>& s, int gl) {
        half8_t xf[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xf[j] = __builtin_bit_cast(half8_t, xs_me[gl * kSlots + j * 4 * TP]);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // B operand that removes the unpack offsets and the zero point: -(1024 + z) under the
            // low-nibble pairs, -(64 + z) under the high-nibble pairs.  One MFMA with it per k32
            // step replaces four packed subtractions per weight word on the vector ALU, which is
            // the unit this kernel saturates; all products are exact and the sums are fp32.
            const half2_t h   = as_half2(s.q[r]);
            const half2_t n64 = half2_t{h[0], h[0]} * half2_t{(half_t)-1.f, (half_t)-1.f};
            const uint32_t zb = ((s.q[r] >> 4) & 0xfu) * 0x10001u + 0xE400E400u;  // -(1024 + z) twice
            half8_t bz;
            bz[0] = as_half2(zb)[0]; bz[1] = as_half2(zb)[1]; bz[2] = n64[0]; bz[3] = n64[1];
            bz[4] = bz[0]; bz[5] = bz[1]; bz[6] = bz[2]; bz[7] = bz[3];
            // Convert the scale now and hide it from the optimiser: otherwise the conversion is
            // folded into the final multiply-add, the Q word stays live past the refill of this
            // stage, and the refill needs a copy that waits for every load in flight.
            float sf = scale_is_normal(s.q[r]) ? (float)h[1] : 0.f;
            asm volatile("" : "+v"(sf));
            float4_t g4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) g4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[j], bz, g4, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t v[4];
                unpack_offset(s.w[r][j], v, uc);
                half8_t wf;
                wf[0] = as_half2(v[0])[0]; wf[1] = as_half2(v[0])[1]; wf[2] = as_half2(v[1])[0]; wf[3] = as_half2(v[1])[1];
                wf[4] = as_half2(v[2])[0]; wf[5] = as_half2(v[2])[1]; wf[6] = as_half2(v[3])[0]; wf[7] = as_half2(v[3])[1];
                g4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[j], wf, g4, 0, 0, 0);
            }
            acc[r] += sf * g4;
        }
    };

    Stage<R> st[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        if (gs0 + d < gs1) load(st[d], gs0 + d);
    }

    for (int done = 0; done < most; done += p.GC) {
        if (done > 0) __syncthreads();  // every wave is finished with the previous chunk
        // ---- stage X[t0 .. t0+TP) for `GC` groups of every slice, in operand order ----
        // Four loads per thread are issued before the first is stored, so that a chunk costs one
        // memory round trip and not one per slice.  Indices past the end repeat the last slot.
        {
            const int lgcs  = p.lgGC + (TP == 4 ? 6 : (TP == 8 ? 7 : 8));  // log2(GC * kSlots)
            const int total = p.Sk << lgcs;
            for (int base = tid; base < total; base += 4 * blockDim.x) {
                u32x4_t tmp[4];
                int     at[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int idx = min(base + u * (int)blockDim.x, total - 1);
                    const int sl  = idx >> lgcs;
                    const int s   = idx & ((1 << lgcs) - 1);
                    const int cc  = s % TP;
                    const int bb  = (s / TP) & 3;
                    const int jj  = (s / (4 * TP)) & 3;
                    const int gl  = s / kSlots;
                    const int sb  = min(G0 + sl * most, G1);       // slice begin
                    const int se  = min(sb + most, G1);            // slice end
                    const int g   = max(min(sb + done + gl, se - 1), 0);  // past the slice: repeat a valid group
                    const int row = min(t0 + cc, T - 1);
                    at[u]  = idx;
                    tmp[u] = *reinterpret_cast<const u32x4_t*>(p.X + (int64_t)row * K + g * kGroup + 32 * jj + 8 * bb);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) xs[at[u]] = tmp[u];
            }
        }
        __syncthreads();
        const int ge = min(gs0 + done + p.GC, gs1);
        int       g  = gs0 + done;
        // steady state: whole rounds whose refills are all in range.  No branch around a load,
        // so the number of loads in flight is known and each stage waits only for its own data.
        bool steady = false;
        // (the compiler-issued loads are all complete here, the X staging above waited for them;
        // saying so keeps the compiler from draining at the loop header)
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        for (; g + kDepth <= ge && g + 2 * kDepth <= gs1; g += kDepth) {
            steady = true;
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                wait_stage(st[d]);
                compute(st[d], g + d - gs0 - done);
                refill(st[d], g + d + kDepth);
            }
        }
        if (steady) {
#pragma unroll
            for (int d = 0; d < kDepth; ++d) wait_all(st[d]);
        }
        // the last one or two rounds of the slice
        for (; g < ge; g += kDepth) {
#pragma unroll
            for (int d = 0; d < kDepth; ++d) {
                if (g + d < ge) {
                    compute(st[d], g + d - gs0 - done);
                    if (g + d + kDepth < gs1) load(st[d], g + d + kDepth);
                }
            }
        }
    }

    // ---- add the slices in LDS, slice order ----
    if (p.Sk > 1) {
        __syncthreads();
        float* red = reinterpret_cast<float*>(xs);  // [Sk][Wn][R][4][64]
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[(((slice * Wn + wn) * R + r) * 4 + i) * 64 + lane] = acc[r][i];
        __syncthreads();
        if (slice != 0 && p.SK == 1) return;
        if (slice == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = 0.f;
                    for (int s = 0; s < p.Sk; ++s) v += red[(((s * Wn + wn) * R + r) * 4 + i) * 64 + lane];
                    acc[r][i] = v;
                }
            }
        }
    }

    // ---- split K across workgroups: exchange partial tiles through the workspace ----
    // The XCDs' L2 caches are not coherent with each other.  Partials and the counter are
    // therefore moved with agent-scope atomic stores/loads (write-through, read-through): a
    // full agent-scope fence would write back and invalidate the whole L2 once per workgroup,
    // which costs far more than the GEMM.  A store's completion (vmcnt reaching zero) means the
    // value has reached memory, so waiting for it before the counter increment orders the two.
    // Only slice 0 holds sums now; the other slices stay for the workgroup barriers.
    if (p.SK > 1) {
        const int64_t zs = (int64_t)blockIdx.z * p.SK;
        if (slice == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float* wp = p.ws + ((zs + split) * NT + nt[r]) * 256 + lane;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (4 * b + i < Tl && nt_first + r < NT)
                        __hip_atomic_store(wp + i * 64, acc[r][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __builtin_amdgcn_s_waitcnt(0);  // all of this wave's stores are complete
        }
        __syncthreads();
        if (tid == 0) {
            int*       cp   = p.cnt + blockIdx.z * gridDim.x + blockIdx.x;
            const int  old  = __hip_atomic_fetch_add(cp, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool last = old == p.SK - 1;
            if (last) __hip_atomic_store(cp, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
            last_flag = last;
        }
        __syncthreads();
        if (!last_flag || slice != 0) return;
        // sum the SK partials in split order; eight splits' loads are in flight at a time (a
        // load-add-load-add chain would pay one memory round trip per split)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};
            for (int s0 = 0; s0 < p.SK; s0 += 8) {
                float v[8][4];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float* wp = p.ws + ((zs + min(s0 + u, p.SK - 1)) * NT + nt[r]) * 256 + lane;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        v[u][i] = __hip_atomic_load(wp + i * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (s0 + u < p.SK) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc[r][i] += v[u][i];
                    }
                }
            }
        }
    }

    // ---- epilogue: lane (c, b) of tile r holds column n = 16*nt + c, tokens t0 + 4b + i ----
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (nt_first + r >= NT) continue;
        const int n = nt[r] * kTileN + c;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half_t h     = (half_t)acc[r][i];
            const int    token = t0 + 4 * b + i;
            if constexpr (EPI == kEpiSilu) {
                // gate = even column, up = odd column: fetch the neighbour lane's value
                const float mine  = (float)h;
                const float other = __shfl_xor(mine, 1);
                if (4 * b + i < Tl && (c & 1) == 0) {
                    const half_t o = (half_t)(mine / (1.f + __expf(-mine)) * other);
                    p.C[(int64_t)token * (N / 2) + (n >> 1)] = __builtin_bit_cast(uint16_t, o);
                }
            }
            else if (4 * b + i < Tl) {
                const int64_t at = (int64_t)token * N + n;
                if constexpr (EPI == kEpiGemm) {
                    p.C[at] = __builtin_bit_cast(uint16_t, h);
                }
                else {
                    const half_t rr = __builtin_bit_cast(half_t, p.Rsd[at]);
                    const half_t o  = (half_t)((float)rr + (float)h);
                    p.C[at]         = __builtin_bit_cast(uint16_t, o);
                }
            }
        }
    }
}

template<int R, int TP, int D>
hipError_t launch_rtd(const DecodeParams& p, dim3 grid, dim3 block, size_t lds, int epilogue, hipStream_t st)
{
#define W4A16_LAUNCH(EPI)                                                                                              \
    do {                                                                                                               \
        auto kfn = decode_kernel<R, TP, D, EPI>;                                                                       \
        if (lds > 64 * 1024) {                                                                                         \
            static std::atomic<uint64_t> raised{0}; /* per instantiation, one bit per device */                        \
            const hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(kfn), (int)kMaxLds, raised);            \
            if (e != hipSuccess) return e;                                                                             \
        }                                                                                                              \
        return launch_kernel(kfn, grid, block, lds, st, p);                                                            \
    } while (0)
    switch (epilogue) {
        case kEpiGemm: W4A16_LAUNCH(kEpiGemm);
        case kEpiSilu: W4A16_LAUNCH(kEpiSilu);
        default: W4A16_LAUNCH(kEpiAdd);
    }
#undef W4A16_LAUNCH
}

template<int R, int D>
hipError_t launch_rd(int tp, const DecodeParams& p, dim3 grid, dim3 block, size_t lds, int epilogue, hipStream_t st)
{
    switch (tp) {
        case 4: return launch_rtd<R, 4, D>(p, grid, block, lds, epilogue, st);
        case 8: return launch_rtd<R, 8, D>(p, grid, block, lds, epilogue, st);
        default: return launch_rtd<R, 16, D>(p, grid, block, lds, epilogue, st);
    }
}

struct Plan {
    int  tp, sk_wg, gc, nb, z;
    bool ok;
};

Plan make_plan(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len)
{
    Plan      pl{};
    const int G = K / kGroup, NT = N / kTileN;
    pl.tp = T <= 4 ? 4 : (T <= 8 ? 8 : 16);
    pl.z  = (T + 15) / 16;
    pl.nb = (NT + cf.wn * cf.r - 1) / (cf.wn * cf.r);
    const long wgs = (long)pl.nb * pl.z;
    int        sk  = 1;
    if (cf.fill > 0) {
        // as many splits as keep the grid within 256 * fill workgroups: one more would start a
        // second, mostly empty round
        const long want = std::max(1l, (long)cf.fill * 256 / wgs);
        sk              = (int)std::max(1l, std::min<long>(want, std::max(1, G / cf.sk)));
        // partial tiles must fit the workspace, counters the counter array
        while (sk > 1 && ((size_t)pl.z * sk * NT * 1024 > ws_bytes || wgs > cnt_len)) --sk;
    }
    pl.sk_wg = sk;
    // longest slice, in groups
    const int per_split = (G + sk - 1) / sk;
    const int most      = (per_split + cf.sk - 1) / cf.sk;
    // groups per slice and staged chunk: a multiple of the pipeline depth such that the
    // activations of all slices fit in LDS
    // (kDepth times a power of two, so that the staging loop needs no division)
    const int fit = (int)(kMaxLds / ((size_t)cf.sk * 256 * pl.tp));
    pl.ok         = fit >= cf.depth && G / sk >= cf.sk && pl.z <= 65535;
    int gc        = cf.depth;
    while (gc < most && gc * 2 <= fit) gc *= 2;
    pl.gc = gc;
    return pl;
}

}  // namespace

bool decode_feasible(const DecodeConfig& cf, int N, int T, int K)
{
    if (N <= 0 || K <= 0 || T <= 0) return false;
    if (N % kTileN != 0 || K % kGroup != 0) return false;
    if (cf.wn * cf.sk > kMaxWaves || cf.wn < 1 || cf.sk < 1 || (cf.wn & (cf.wn - 1)) != 0) return false;
    if (!((cf.r == 1 && (cf.depth == 4 || cf.depth == 8)) || (cf.r == 2 && cf.depth == 4))) return false;
    return make_plan(cf, N, T, K, 0, 0).ok;
}

size_t decode_scratch_bytes(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len)
{
    const Plan pl = make_plan(cf, N, T, K, ws_bytes, cnt_len);
    return pl.sk_wg > 1 ? (size_t)pl.z * pl.sk_wg * (N / kTileN) * 1024 : 0;
}

int decode_grid(const DecodeConfig& cf, int N, int T, int K, size_t ws_bytes, int cnt_len)
{
    const Plan pl = make_plan(cf, N, T, K, ws_bytes, cnt_len);
    return pl.nb * pl.sk_wg * pl.z;
}

hipError_t decode_launch(const DecodeConfig& cf, const GemmArgs& a, float* ws, size_t ws_bytes, int* cnt, int cnt_len,
                         hipStream_t st)
{
    if (!ws || !cnt) {
        ws_bytes = 0;
        cnt_len  = 0;
    }
    const Plan   pl = make_plan(cf, a.N, a.T, a.K, ws_bytes, cnt_len);
    int lg = 0;
    while ((1 << lg) < cf.wn) ++lg;
    int lgc = 0;
    while ((1 << lgc) < pl.gc) ++lgc;
    const int    G         = a.K / kGroup;
    const int    per_split = (G + pl.sk_wg - 1) / pl.sk_wg;
    const int    per_slice = (per_split + cf.sk - 1) / cf.sk;
    DecodeParams p{a.C, reinterpret_cast<const u32x4_t*>(a.A), a.X, a.Q, a.R, ws, cnt, a.N, a.T, a.K,
                   cf.wn, lg, cf.sk, pl.sk_wg, pl.gc, lgc, per_split, per_slice};
    const dim3   grid(pl.nb, pl.sk_wg, pl.z), block(64 * cf.wn * cf.sk);
    const size_t x_bytes   = (size_t)cf.sk * pl.gc * 256 * pl.tp;
    const size_t red_bytes = cf.sk > 1 ? (size_t)cf.sk * cf.wn * cf.r * 1024 : 0;
    const size_t lds       = std::max(x_bytes, red_bytes);
    if (cf.r == 2) return launch_rd<2, 4>(pl.tp, p, grid, block, lds, a.epilogue, st);
    if (cf.depth == 4) return launch_rd<1, 4>(pl.tp, p, grid, block, lds, a.epilogue, st);
    return launch_rd<1, 8>(pl.tp, p, grid, block, lds, a.epilogue, st);
}

}  // namespace w4a16
