// Decode (skinny) W4A16 GEMM for gfx950: up to 16 tokens per workgroup column.
//
// A workgroup owns R adjacent 16-column weight tiles and ALL of K.  Its S waves each take
// a contiguous slice of the K/128 quantisation groups ("sliced K"), so every wave streams
// whole 1 KiB weight tiles from HBM with one 128-bit load per lane, keeps kDepth tiles in
// flight, and the slice partials are summed in LDS in a fixed order (deterministic; no
// cross-workgroup exchange, no atomics).
//
// Per group a wave computes, for its 16 columns, accg[t, n] = sum_k X[t, k] * (q[k, n] - z[n])
// with four v_mfma_f32_16x16x32_f16 (activations as the A operand, de-offset int4 as the B
// operand; the differences are exact in fp16), then acc += s[n] * accg in fp32.  Scaling
// after the group sum moves the per-weight multiply out of the inner loop: the dequantise
// costs 9 VALU instructions per 8 weights.  The result differs from "round every weight to
// fp16 first" only by that rounding (<= 2^-11 relative per term).
#include "w4a16_common.h"
#include "w4a16_internal.h"

namespace w4a16 {

namespace {

// weight tiles in flight per wave and column tile, bounded by the 128-VGPR budget of a
// 1024-thread workgroup
constexpr int depth_for(int r)
{
    return r == 1 ? 4 : (r == 2 ? 3 : 2);
}

template<int R>
struct Stage {
    u32x4_t  w[R];
    uint32_t q[R];
    u32x4_t  x[4];
};

template<int R, int EPI, int kDepth = depth_for(R)>
__global__ void __launch_bounds__(R == 4 ? 512 : 1024)
decode_kernel(uint16_t* __restrict__ C, const u32x4_t* __restrict__ A, const uint16_t* __restrict__ X,
              const uint32_t* __restrict__ Q, const uint16_t* R_, int N, int T, int K)
{
    extern __shared__ float red[];  // [S][R][4][64]

    const int lane  = threadIdx.x & 63;
    const int slice = threadIdx.x >> 6;
    const int S     = blockDim.x >> 6;
    const int c     = lane & 15;
    const int b     = lane >> 4;
    const int G     = K / kGroup;
    const int nt0   = blockIdx.x * R;
    const int t0    = blockIdx.y * 16;

    const int g0 = (int)((int64_t)slice * G / S);
    const int g1 = (int)((int64_t)(slice + 1) * G / S);

    const u32x4_t*  Ap = A + ((int64_t)nt0 * G) * 64 + lane;  // + (r*G + g) * 64
    const uint32_t* Qp = Q + nt0 * kTileN + c;                // + g*N + r*16
    // Rows of the MFMA's A operand are independent, and output rows >= T are never stored, so
    // lanes whose token does not exist just re-read the last valid row.
    const int       xrow = min(t0 + c, T - 1);
    const uint16_t* Xp   = X + (int64_t)xrow * K + 8 * b;  // + g*128 + 32*j
    const UnpackConsts uc;

    auto load = [&](Stage<R>& s, int g) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            s.w[r] = __builtin_nontemporal_load(Ap + ((int64_t)r * G + g) * 64);
            s.q[r] = Qp[(int64_t)g * N + r * kTileN];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s.x[j] = *reinterpret_cast<const u32x4_t*>(Xp + g * kGroup + 32 * j);
        }
    };

    float4_t acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = float4_t{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](const Stage<R>& s) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            half2_t z1024, z64;
            half_t  sc;
            split_q(s.q[r], z1024, z64, sc);
            const uint32_t w[4] = {s.w[r][0], s.w[r][1], s.w[r][2], s.w[r][3]};
            float4_t       g4   = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half8_t wf = dequant_sub(w[j], z1024, z64, uc);
                const half8_t xf = __builtin_bit_cast(half8_t, s.x[j]);
                g4               = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf, wf, g4, 0, 0, 0);
            }
            const float sf = (float)sc;
            acc[r] += sf * g4;
        }
    };

    Stage<R> st[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        if (g0 + d < g1) load(st[d], g0 + d);
    }
    for (int g = g0; g < g1; g += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (g + d < g1) {
                compute(st[d]);
                if (g + d + kDepth < g1) load(st[d], g + d + kDepth);
            }
        }
    }

    // ---- sum the K slices in LDS, fixed order ----
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((slice * R + r) * 4 + i) * 64 + lane] = acc[r][i];
    }
    __syncthreads();

    for (int e = threadIdx.x; e < 128 * R; e += blockDim.x) {
        const int r     = e >> 7;
        const int t     = (e >> 3) & 15;
        const int p     = e & 7;
        const int token = t0 + t;
        if (token >= T) continue;
        const int l0 = 16 * (t >> 2) + 2 * p;
        const int i  = t & 3;
        float     y0 = 0.f, y1 = 0.f;
        for (int s = 0; s < S; ++s) {
            const float2 v = *reinterpret_cast<const float2*>(&red[((s * R + r) * 4 + i) * 64 + l0]);
            y0 += v.x;
            y1 += v.y;
        }
        const int     n  = (nt0 + r) * kTileN + 2 * p;
        const half_t  h0 = (half_t)y0, h1 = (half_t)y1;
        if constexpr (EPI == kEpiGemm) {
            *reinterpret_cast<uint32_t*>(C + (int64_t)token * N + n) = as_u32(half2_t{h0, h1});
        }
        else if constexpr (EPI == kEpiSilu) {
            const float  gt = (float)h0, up = (float)h1;
            const float  v  = gt / (1.f + __expf(-gt)) * up;
            const half_t o  = (half_t)v;
            C[(int64_t)token * (N / 2) + (n >> 1)] = __builtin_bit_cast(uint16_t, o);
        }
        else {
            const half2_t rr = as_half2(*reinterpret_cast<const uint32_t*>(R_ + (int64_t)token * N + n));
            const half_t  o0 = (half_t)((float)rr[0] + (float)h0);
            const half_t  o1 = (half_t)((float)rr[1] + (float)h1);
            *reinterpret_cast<uint32_t*>(C + (int64_t)token * N + n) = as_u32(half2_t{o0, o1});
        }
    }
}

template<int R>
hipError_t launch_r(int s, const GemmArgs& a, hipStream_t st)
{
    const dim3   grid(a.N / kTileN / R, (a.T + 15) / 16);
    const dim3   block(64 * s);
    const size_t lds = (size_t)s * R * 1024;
    const u32x4_t* A4 = reinterpret_cast<const u32x4_t*>(a.A);
    switch (a.epilogue) {
        case kEpiGemm:
            hipLaunchKernelGGL((decode_kernel<R, kEpiGemm>), grid, block, lds, st, a.C, A4, a.X, a.Q, a.R, a.N, a.T,
                               a.K);
            break;
        case kEpiSilu:
            hipLaunchKernelGGL((decode_kernel<R, kEpiSilu>), grid, block, lds, st, a.C, A4, a.X, a.Q, a.R, a.N, a.T,
                               a.K);
            break;
        default:
            hipLaunchKernelGGL((decode_kernel<R, kEpiAdd>), grid, block, lds, st, a.C, A4, a.X, a.Q, a.R, a.N, a.T,
                               a.K);
            break;
    }
    return hipGetLastError();
}

}  // namespace

bool decode_feasible(int r, int s, int N, int T, int K)
{
    if (N <= 0 || K <= 0 || T <= 0) return false;
    if (N % (kTileN * r) != 0 || K % kGroup != 0) return false;
    if (s < 1 || s > (r == 4 ? 8 : 16) || s > K / kGroup) return false;
    if ((T + 15) / 16 > 65535) return false;
    return r == 1 || r == 2 || r == 4;
}

int decode_grid(int r, int s, int N, int T, int K)
{
    (void)s;
    (void)K;
    return (N / kTileN / r) * ((T + 15) / 16);
}

hipError_t decode_launch(int r, int s, const GemmArgs& a, hipStream_t st)
{
    switch (r) {
        case 1: return launch_r<1>(s, a, st);
        case 2: return launch_r<2>(s, a, st);
        default: return launch_r<4>(s, a, st);
    }
}

}  // namespace w4a16
