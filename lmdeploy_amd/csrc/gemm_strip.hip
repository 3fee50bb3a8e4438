// Decode (skinny) W4A16 GEMM for gfx950, "strip" decomposition: bound by HBM.
//
// The weight matrix is a grid of 1 KiB tiles (16 columns x one 128-row quantisation group).
// The column tiles are dealt out as evenly as possible to B workgroups, B a multiple of the CU
// count: workgroup b owns a strip of R or R-1 adjacent column tiles over the whole of K.  Its
// eight waves (sixteen for one-tile strips at up to eight tokens) deal the groups of K out
// round-robin; a wave walks its groups and, per group, loads the strip's R tiles (R KiB contiguous
// in the group-major tile layout) and its own activations of that group straight into registers -
// no cooperative staging, no barrier and no other wave involved until the end, when the partial
// strips are added in LDS in slice order.
//
// Why this shape: (a) every CU gets the same number of tiles to within one strip column, which
// the column-block decomposition could not offer for matrices like 4096 x 22016 (1376 column
// tiles); (b) the activations of a group are loaded once per wave and used for R tiles, instead of
// a workgroup-wide LDS staging round trip with two barriers per chunk - at 16 tokens that staging
// cost more than a third of the kernel; (c) two groups are in
// flight per wave from its first instruction on (2 R + 8 KiB).
//
// With 32 tokens per workgroup (17 to 32 tokens) every workgroup still reads all of the activations
// once, which is then several times the weight bytes of a narrow strip: the activations of a group go
// from memory straight into the wave's LDS patch (no registers), which leaves registers for strips of
// up to eight tiles, so that one workgroup per CU suffices on the widest matrices and the activations
// are read 256 times instead of 512.
//
// Arithmetic per group and tile is that of the column-block decode kernel: four MFMAs on the
// unpacked int4 still carrying its fp16 offset, four on a B operand of -(offset + z), then
// acc += s * sum in fp32.
#include "strip_body.h"

#include <algorithm>

namespace w4a16 {

namespace {

using namespace strip;

// RMAX = width of the wide strips (base + 1 when the column tiles do not divide evenly).
// D = groups in flight per wave (2, or 1 for wide strips: see strip_launch).
template<int RMAX, int TP, int EPI, int D = 2>
__global__ void __launch_bounds__(64 * kWaves) strip_kernel(const StripParams p)
{
    extern __shared__ __attribute__((aligned(16))) u32x4_t smem[];  // activation patches [8][1 or 2][TP][16], then sums [8][R][H][64]
    clock_record_start(p.clk, blockIdx.x == gridDim.x / 2 && blockIdx.y == 0 && threadIdx.x == 0);
    for (int pass = 0; pass < p.passes; ++pass) {
        const int  bx   = pass * gridDim.x + blockIdx.x;
        const bool wide = bx < p.rem;
        const int  col0 = bx * p.base + min(bx, p.rem);
        if (pass) __syncthreads();  // the sums of the previous strip have been read out of LDS
        bool done = false;
        if constexpr (RMAX > 1) {
            if (!wide && p.base == RMAX - 1) {
                strip_body<RMAX - 1, TP, EPI, false, kWaves, NoWait, 1, D>(p, col0, smem);
                done = true;
            }
        }
        if (!done) strip_body<RMAX, TP, EPI, false, kWaves, NoWait, 1, D>(p, col0, smem);
    }
    clock_record_stop(p.clk, blockIdx.x == gridDim.x / 2 && blockIdx.y == 0 && threadIdx.x == 0);
}

// One-tile strips at up to eight tokens: sixteen waves instead of eight, so that a wave walks half as many groups
// one after the other and the CU has 32 KiB of weights requested instead of 16 (7B down at one token: 8.6 -> 7.6 us,
// o: 4.65 -> 4.5).  At five to eight tokens the activation rows double what a stage holds, and each wave keeps one
// group in flight instead of two (down at eight tokens 9.7 -> 9.1 us, o 5.0 -> 4.85); at sixteen tokens, and for
// two-tile strips, eight waves are ahead.
constexpr int kWavesNarrow = 16;
template<int TP, int EPI, int D>
__global__ void __launch_bounds__(64 * kWavesNarrow) strip_kernel_narrow(const StripParams p)
{
    extern __shared__ __attribute__((aligned(16))) u32x4_t smem[];
    clock_record_start(p.clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
    strip_body<1, TP, EPI, false, kWavesNarrow, NoWait, 1, D>(p, (int)blockIdx.x, smem);
    clock_record_stop(p.clk, blockIdx.x == gridDim.x / 2 && threadIdx.x == 0);
}

template<int TP, int D>
hipError_t launch_narrow(const StripParams& p, dim3 grid, int epilogue, hipStream_t st)
{
    const dim3   block(64 * kWavesNarrow);
    const size_t lds = (size_t)kWavesNarrow * std::max(1024, TP * 256);
    switch (epilogue) {
        case kEpiGemm: return launch_kernel(strip_kernel_narrow<TP, kEpiGemm, D>, grid, block, lds, st, p);
        case kEpiSilu: return launch_kernel(strip_kernel_narrow<TP, kEpiSilu, D>, grid, block, lds, st, p);
        default: return launch_kernel(strip_kernel_narrow<TP, kEpiAdd, D>, grid, block, lds, st, p);
    }
}

// The same kernel for group sizes 64 and 32 (NQ = 2, 4 quantisation groups per 128-row tile): 16 token rows per
// workgroup whatever the token count, the epilogue chosen at run time, strips of at most kMaxRQ tiles (a tile
// brings NQ scale words along) - eight instantiations instead of ninety-six.
constexpr int kMaxRQ = 4;
template<int RMAX, int NQ>
__global__ void __launch_bounds__(64 * kWaves) strip_kernel_q(const StripParams p)
{
    extern __shared__ __attribute__((aligned(16))) u32x4_t smem[];
    for (int pass = 0; pass < p.passes; ++pass) {
        const int  bx   = pass * gridDim.x + blockIdx.x;
        const bool wide = bx < p.rem;
        const int  col0 = bx * p.base + min(bx, p.rem);
        if (pass) __syncthreads();
        bool done = false;
        if constexpr (RMAX > 1) {
            if (!wide && p.base == RMAX - 1) {
                strip_body<RMAX - 1, 16, kEpiRuntime, false, kWaves, NoWait, NQ>(p, col0, smem);
                done = true;
            }
        }
        if (!done) strip_body<RMAX, 16, kEpiRuntime, false, kWaves, NoWait, NQ>(p, col0, smem);
    }
}

template<int NQ>
hipError_t launch_q(int rmax, const StripParams& p, dim3 grid, size_t lds, hipStream_t st)
{
    const dim3 block(64 * kWaves);
    switch (rmax) {
        case 1: return launch_kernel(strip_kernel_q<1, NQ>, grid, block, lds, st, p);
        case 2: return launch_kernel(strip_kernel_q<2, NQ>, grid, block, lds, st, p);
        case 3: return launch_kernel(strip_kernel_q<3, NQ>, grid, block, lds, st, p);
        default: return launch_kernel(strip_kernel_q<4, NQ>, grid, block, lds, st, p);
    }
}

constexpr int kMinRShallow = 3;  // narrowest strip that exists with one group in flight per wave
template<int RMAX, int TP, int D = 2>
hipError_t launch_rt(const StripParams& p, dim3 grid, size_t lds, int epilogue, hipStream_t st)
{
    const dim3 block(64 * kWaves);
#define W4A16_LAUNCH(EPI)                                                                                              \
    do {                                                                                                               \
        auto kfn = strip_kernel<RMAX, TP, EPI, D>;                                                                     \
        if constexpr (TP == 32) { /* up to 128 KiB of LDS: above the default limit */                                  \
            static std::atomic<uint64_t> raised{0};                                                                    \
            const hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(kfn), 8 * kMaxR32 * 2 * 1024, raised);  \
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

template<int RMAX>
hipError_t launch_r(int tp, int depth, const StripParams& p, dim3 grid, size_t lds, int epilogue, hipStream_t st)
{
    if constexpr (RMAX >= kMinRShallow) {
        if (depth == 1) {
            switch (tp) {
                case 4: return launch_rt<RMAX, 4, 1>(p, grid, lds, epilogue, st);
                case 8: return launch_rt<RMAX, 8, 1>(p, grid, lds, epilogue, st);
                case 16: return launch_rt<RMAX, 16, 1>(p, grid, lds, epilogue, st);
                default:
                    if constexpr (RMAX <= kMaxR32) return launch_rt<RMAX, 32, 1>(p, grid, lds, epilogue, st);
                    break;
            }
        }
    }
    switch (tp) {
        case 4: return launch_rt<RMAX, 4>(p, grid, lds, epilogue, st);
        case 8: return launch_rt<RMAX, 8>(p, grid, lds, epilogue, st);
        case 16: return launch_rt<RMAX, 16>(p, grid, lds, epilogue, st);
        default:
            // 32 tokens per block: twice the accumulators and activation registers, strips of at most kMaxR32 tiles
            if constexpr (RMAX <= kMaxR32) return launch_rt<RMAX, 32>(p, grid, lds, epilogue, st);
            return hipErrorInvalidValue;
    }
}

struct StripPlan {
    int  strips, base, rem, rmax, passes;
    bool ok;
};
constexpr int kInPasses = 3;  // value of `per_cu` that asks for one workgroup per CU walking several strips in turn

// `per_cu` strips per CU are aimed for; more if a strip would otherwise be wider than the limit.
// block_t = tokens per workgroup: 16 (activation rows padded down to 4 or 8 for fewer tokens) or 32.
// Compute units of the current device (the strips are dealt to that many workgroups, or a multiple): asked
// once per device; 256, MI355X's count, where no device can be asked.
int device_cus()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return kNumCU;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = kNumCU;
    cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

StripPlan make_plan(int per_cu, int block_t, int N, int T, int K, int maxr_limit = kMaxR)
{
    const int cus = device_cus();
    StripPlan pl{};
    if (N <= 0 || K <= 0 || T <= 0 || N % kTileN != 0 || K % kGroup != 0 || per_cu < 1) return pl;
    if (block_t != 16 && block_t != 32) return pl;
    if (block_t == 32 && T <= 16) return pl;  // the 16-token kernel covers these
    const int NT   = N / kTileN;
    const int maxr = std::min(maxr_limit, block_t == 32 ? kMaxR32 : kMaxR);
    int       m    = per_cu == kInPasses ? 1 : per_cu;
    while ((NT + cus * m - 1) / (cus * m) > maxr) ++m;
    pl.strips = std::min(NT, cus * m);
    pl.base   = NT / pl.strips;
    pl.rem    = NT % pl.strips;
    pl.rmax   = pl.base + (pl.rem ? 1 : 0);
    pl.passes = 1;
    // 32-bit per-lane offsets into X; grid limits
    pl.ok = (int64_t)T * K * 2 < (1ll << 32) && (T + block_t - 1) / block_t <= 65535 &&
            (per_cu == 1 || pl.strips == cus * m);
    if (per_cu == kInPasses) {
        // Matrices too wide for one strip per CU: instead of m workgroups per CU side by side (16 or more waves
        // per CU asking for memory at once), one workgroup per CU takes its m strips in turn.  A plain streaming
        // read of 244 MiB is 10 % faster from 8 waves per CU than from 16.
        pl.ok     = pl.ok && m >= 2;
        pl.passes = m;
        pl.strips = cus;  // workgroups; base and rem still describe all m * cus strips
    }
    return pl;
}

}  // namespace

bool strip_feasible(int per_cu, int block_t, int N, int T, int K)
{
    return make_plan(per_cu, block_t, N, T, K).ok;
}

int strip_grid(int per_cu, int block_t, int N, int T, int K)
{
    const StripPlan pl = make_plan(per_cu, block_t, N, T, K);
    return pl.strips * ((T + block_t - 1) / block_t);  // (workgroups)
}

int strip_width(int per_cu, int block_t, int N, int T, int K)
{
    return make_plan(per_cu, block_t, N, T, K).rmax;
}

hipError_t strip_launch(int per_cu, int block_t, const GemmArgs& a, hipStream_t st)
{
    const StripPlan pl = make_plan(per_cu, block_t, a.N, a.T, a.K);
    if (!pl.ok) return hipErrorInvalidValue;
    const int   tp = block_t == 32 ? 32 : (a.T <= 4 ? 4 : (a.T <= 8 ? 8 : 16));
    const int   h  = tp > 16 ? tp / 16 : 1;
    StripParams p{a.C, reinterpret_cast<const u32x4_t*>(a.A), a.X, a.Q, a.R, a.N, a.T, a.K, pl.base, pl.rem,
                  a.epilogue, pl.passes, a.clk};
    const dim3   grid(pl.strips, (a.T + block_t - 1) / block_t);
    // per wave: the sums of its strip, over its activation patch(es) - two for 32 tokens, which arrive straight from memory
    const size_t lds = (size_t)kWaves * std::max(pl.rmax * h * 1024, tp * 256 * (tp >= kDmaTokens ? 2 : 1));
    if (tp <= 8 && pl.rmax == 1 && pl.passes == 1 && a.K / kGroup >= 2 * kWavesNarrow)
        return tp == 4 ? launch_narrow<4, 2>(p, grid, a.epilogue, st) : launch_narrow<8, 1>(p, grid, a.epilogue, st);
    // Two groups per wave in flight are waves x 2 x R KiB per CU.  The memory system streams fastest with 32 - 64 KiB
    // requested per CU (more is slower); beyond that every wave keeps one group in flight instead: 7B gate_up
    // 12.9 -> 12.2 us at 16 tokens (strips of 6), 16.9 -> 15.7 at 32, and 11.4 -> 11.2 at one (two workgroups of 3 per
    // CU), 70B gate_up 44.8 -> 43.5; narrower strips lose (qkv, strips of 3: 7.4 -> 8.0).
    const int waves_per_cu = kWaves * ((pl.strips + device_cus() - 1) / device_cus());
    const int depth        = waves_per_cu * 2 * pl.rmax > 64 ? 1 : 2;
    switch (pl.rmax) {
        case 1: return launch_r<1>(tp, depth, p, grid, lds, a.epilogue, st);
        case 2: return launch_r<2>(tp, depth, p, grid, lds, a.epilogue, st);
        case 3: return launch_r<3>(tp, depth, p, grid, lds, a.epilogue, st);
        case 4: return launch_r<4>(tp, depth, p, grid, lds, a.epilogue, st);
        case 5: return launch_r<5>(tp, depth, p, grid, lds, a.epilogue, st);
        case 6: return launch_r<6>(tp, depth, p, grid, lds, a.epilogue, st);
        case 7: return launch_r<7>(tp, depth, p, grid, lds, a.epilogue, st);
        default: return launch_r<8>(tp, depth, p, grid, lds, a.epilogue, st);
    }
}

// Group sizes 64 and 32: strips of up to kMaxRQ tiles, one workgroup per strip (as many workgroups per CU as that
// takes), token blocks of 16 side by side in the grid for more than 16 tokens (each block streams the weights again).
bool strip_groups_feasible(int nq, int N, int T, int K)
{
    return (nq == 2 || nq == 4) && make_plan(1, 16, N, T, K, kMaxRQ).ok;
}

hipError_t strip_groups_launch(int nq, const GemmArgs& a, hipStream_t st)
{
    const StripPlan pl = make_plan(1, 16, a.N, a.T, a.K, kMaxRQ);
    if (!pl.ok || (nq != 2 && nq != 4)) return hipErrorInvalidValue;
    StripParams  p{a.C, reinterpret_cast<const u32x4_t*>(a.A), a.X, a.Q, a.R, a.N, a.T, a.K, pl.base, pl.rem,
                   a.epilogue, pl.passes};
    const dim3   grid(pl.strips, (a.T + 15) / 16);
    const size_t lds = (size_t)kWaves * std::max(pl.rmax * 1024, 16 * 256);
    return nq == 2 ? launch_q<2>(pl.rmax, p, grid, lds, st) : launch_q<4>(pl.rmax, p, grid, lds, st);
}

}  // namespace w4a16
