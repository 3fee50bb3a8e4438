// The C ABI of libw4a16.so: argument validation, kernel selection, timing and error
// reporting.  No kernel code lives here.
#include "../../include/w4a16.h"
#include "../../include/w4a16_probe.h"
#include "w4a16_internal.h"

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <map>
#include <tuple>
#include <vector>

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    return fail(W4A16_EHIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

bool aligned8(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 7u) == 0;
}

// Group sizes with kernels: the reference's 128 (gemm_s4_f16.cu:243-245 instantiates nothing else and leaves a
// "TODO: add more group sizes"), plus 64 and 32.  Anything else gets the reference's error (gemm_s4_f16.cu:119).
bool group_ok(int group_size)
{
    return group_size == 128 || group_size == 64 || group_size == 32;
}

}  // namespace

struct w4a16_handle {
    hipEvent_t     ev_start{};
    hipEvent_t     ev_end{};
    int            device{};
    w4a16::Scratch scratch{};
    int*           sync{};        // counters of the device-wide barrier of w4a16_gemm_sequence
    int            cus{};         // compute units of the device: workgroups of a persistent launch
    long long      clock_khz{};   // rate of the device's wall clock
    long long      spin_ticks{};  // time limit of one barrier wait
    unsigned long long* clk{};    // measurement aid: cycle, tick and launch counters of w4a16_probe_clock_*
    bool           clk_on{};      // strip kernels and probes launched through this handle record into them
    // fastest kernel found by w4a16_measure, per (n_out, tokens, k); consulted before the heuristic
    std::map<std::tuple<int, int, int>, int> tuned;
};

namespace w4a16 {

// ---- kernel table (the counterpart of the 17 GemmKernel objects of gemm_s4_f16.cu:72-93) ----
namespace {

std::vector<Algo> build_table()
{
    std::vector<Algo> t;
    const int rd[3][2]   = {{1, 8}, {1, 4}, {2, 4}};                                                 // r, depth
    const int wnsk[9][2] = {{8, 1}, {8, 2}, {4, 1}, {4, 2}, {4, 4}, {2, 4}, {2, 8}, {1, 8}, {1, 16}};  // wn, sk
    for (auto& a : rd)
        for (auto& b : wnsk) t.push_back(Algo{0, 16 * a[0] * b[0], 16, b[1], 0, DecodeConfig{a[0], b[0], b[1], a[1], 0}});
    // with K split across workgroups as well
    for (int fill : {1, 2, 4}) {
        t.push_back(Algo{0, 128, 16, 1, 0, DecodeConfig{1, 8, 1, 4, fill}});
        t.push_back(Algo{0, 64, 16, 1, 0, DecodeConfig{1, 4, 1, 4, fill}});
        t.push_back(Algo{0, 128, 16, 2, 0, DecodeConfig{1, 8, 2, 4, fill}});
    }
    // strips of column tiles over the whole of K, 1 or 2 per CU
    // (3: one workgroup per CU that walks several strips in turn, for matrices wider than 8 x 256 column tiles)
    for (int per_cu : {1, 2, 3}) t.push_back(Algo{2, 0, 16, 8, per_cu, DecodeConfig{}});
    // the same with 32 tokens per workgroup (17 tokens and more): half the passes over the weights
    for (int per_cu : {1, 2}) t.push_back(Algo{2, 0, 32, 8, per_cu, DecodeConfig{}});
    for (int v = 0; v < prefill_variants(); ++v) {
        int tn = 0, tt = 0;
        prefill_tile(v, tn, tt);
        t.push_back(Algo{1, tn, tt, 1, v, DecodeConfig{}});
    }
    // the same tiles with K split across 2, 4 or 8 workgroups (few tokens: too few tiles to fill the chip)
    for (int splits : {2, 4, 8}) {
        for (int v = 0; v < prefill_variants(); ++v) {
            int tn = 0, tt = 0;
            prefill_tile(v, tn, tt);
            if (tt <= 128) t.push_back(Algo{1, tn, tt, splits, v, DecodeConfig{}});
        }
    }
    return t;
}

const std::vector<Algo>& table()
{
    static const std::vector<Algo> t = build_table();
    return t;
}

}  // namespace

int algo_count()
{
    return (int)table().size();
}

const Algo& algo_at(int id)
{
    return table()[id];
}

bool algo_feasible(int id, int N, int T, int K, const Scratch& lim)
{
    const Algo& a = algo_at(id);
    if (a.kind == 2) return strip_feasible(a.param, a.tile_t, N, T, K);
    return a.kind == 0 ? decode_feasible(a.dc, N, T, K) :
                         prefill_feasible(a.param, a.slices, N, T, K, lim.ws_bytes, lim.cnt_len);
}

size_t algo_scratch_bytes(int id, int N, int T, int K, const Scratch& lim)
{
    const Algo& a = algo_at(id);
    if (a.kind == 2) return 0;
    return a.kind == 0 ? decode_scratch_bytes(a.dc, N, T, K, lim.ws_bytes, lim.cnt_len) :
                         prefill_scratch_bytes(a.param, a.slices, N, T, K);
}

int algo_grid(int id, int N, int T, int K, const Scratch& sc)
{
    const Algo& a = algo_at(id);
    if (a.kind == 2) return strip_grid(a.param, a.tile_t, N, T, K);
    return a.kind == 0 ? decode_grid(a.dc, N, T, K, sc.ws_bytes, sc.cnt_len) : prefill_grid(a.param, a.slices, N, T, K);
}

hipError_t algo_launch(int id, const GemmArgs& g, const Scratch& sc, hipStream_t st)
{
    const Algo& a = algo_at(id);
    if (a.kind == 2) return strip_launch(a.param, a.tile_t, g, st);
    return a.kind == 0 ? decode_launch(a.dc, g, sc.ws, sc.ws_bytes, sc.cnt, sc.cnt_len, st) :
                         prefill_launch(a.param, a.slices, g, sc, st);
}

// Heuristic choice (the counterpart of Estimate, gemm_s4_f16.cu:184-206).  Above 16 tokens:
// every MFMA prefill tile, unsplit and with K split 2, 4 or 8 ways, is priced with a model of
// measured step times, and so is the decode kernel (which re-reads the weights once per 16
// tokens); the cheapest wins.  Up to 16 tokens: the decode kernel, see below.
int algo_pick(int N, int T, int K, const Scratch& lim)
{
    if (T <= 0 || N <= 0 || K <= 0) return -1;
    if (T > 16) {
        int    best = -1;
        double best_us = 0;
        for (int id = 0; id < algo_count(); ++id) {
            const Algo& a = algo_at(id);
            if (a.kind != 1 || !algo_feasible(id, N, T, K, lim)) continue;
            const double us = prefill_estimate_us(a.param, a.slices, N, T, K);
            if (best < 0 || us < best_us) best = id, best_us = us;
        }
        // decode: launch + the weight stream once per block of 16 tokens; later blocks find part of it
        // in the caches (exponent fitted to 2 .. 8 blocks on Llama-7B shapes)
        // (narrow matrices use the column-block kernel with K split across workgroups: 1.4 x)
        const double blocks    = (T + 15) / 16;
        const double decode_us = 3.0 + std::pow(blocks, 0.85) * ((double)K * N / 2) / 4.2e6 * (N / 16 < 512 ? 1.4 : 1.0);
        // 17..32 tokens: the strip kernel with 32 tokens per workgroup streams the weights once, at
        // 1.2 x (17 tokens) to 1.4 x (32 tokens) the cost of a 16-token pass
        int    strip32 = -1;
        double strip32_us = 0;
        if (T <= 32) {
            for (int id = 0; id < algo_count() && strip32 < 0; ++id) {
                const Algo& a = algo_at(id);
                if (a.kind == 2 && a.tile_t == 32 && a.param == 1 && algo_feasible(id, N, T, K, lim)) strip32 = id;
            }
            strip32_us = 3.0 + (1.2 + 0.2 * (T - 16) / 16.0) * ((double)K * N / 2) / 4.2e6;
        }
        if (best >= 0 && best_us < decode_us && (strip32 < 0 || best_us < strip32_us)) return best;
        if (strip32 >= 0 && strip32_us < decode_us) return strip32;
    }
    // Decode.  Strips of column tiles over the whole of K, one per CU, were the fastest on every
    // Llama-7B/70B shape measured at 1..16 tokens; two narrower strips per CU are slightly ahead on
    // very wide matrices while the activations are small (up to 4 tokens: 7B gate_up 11.5 against 12.0 us at
    // one token, 13.2 against 12.4 at eight - a wide strip shares the sums of its activations among more tiles).  Matrices with too few column tiles to
    // give every CU a strip fall back to the column-block kernel, which can also split K across
    // workgroups.
    // Above 16 tokens every workgroup re-reads the weights once per 16-token block, and narrow
    // matrices are better off splitting K across workgroups (column-block kernel with `fill`).
    if (N / 16 >= 128 && (T <= 16 || N / 16 >= 512)) {
        // (3 = one workgroup per CU taking several strips in turn: only feasible, and then measured 2 - 6 % ahead, for
        // matrices too wide for one strip per CU, such as the 57344 columns of Llama-2-70B's gate_up)
        const int want = (N / 16 >= 1024 && T <= 4) ? 2 : 1;
        for (int per_cu : {3, want, 1}) {
            for (int id = 0; id < algo_count(); ++id) {
                const Algo& a = algo_at(id);
                if (a.kind == 2 && a.tile_t == 16 && a.param == per_cu && algo_feasible(id, N, T, K, lim)) return id;
            }
        }
    }
    // Column-block kernel: one column tile per wave, four groups in flight.  Wide matrices give
    // every wave its own column tiles and share the activations among eight waves; narrow ones
    // also slice K inside the workgroup so that at least 256 workgroups exist.
    const int nt = N / 16, groups = K / 128;
    int       wn, sk, fill = 0;
    if (nt >= 1024) {
        wn = 8, sk = 1;
    }
    else if (nt >= 512) {
        wn = 4, sk = 2;
    }
    else if (T > 8 || (T > 4 && groups >= 64)) {
        // narrow matrix, many tokens: the activations dominate the traffic unless eight waves
        // share them, so K is split across workgroups instead of inside them
        wn = 8, sk = 1, fill = 1;
    }
    else {
        wn = 1, sk = 8;
    }
    for (int id = 0; id < algo_count(); ++id) {
        const Algo& a = algo_at(id);
        if (a.kind == 0 && a.dc.r == 1 && a.dc.depth == 4 && a.dc.wn == wn && a.dc.sk == sk && a.dc.fill == fill &&
            algo_feasible(id, N, T, K, lim))
            return id;
    }
    for (int id = 0; id < algo_count(); ++id)
        if (algo_feasible(id, N, T, K, lim)) return id;
    return -1;
}

}  // namespace w4a16

using namespace w4a16;

namespace {

// Validates the arguments of a GEMM without touching the GPU: < 0 error, 1 nothing to do, 0 go on.
int check_gemm_args(const void* C, const void* A, const void* X, const void* Q, const void* R, int n_out, int tokens,
                    int k, int group_size, int epilogue)
{
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (epilogue < W4A16_GEMM || epilogue > W4A16_FUSED_ADD) return fail(W4A16_EARG, "unknown epilogue %d", epilogue);
    if (n_out < 0 || tokens < 0 || k < 0) return fail(W4A16_EARG, "negative size");
    if (tokens == 0 || n_out == 0) return 1;  // nothing to do
    if (!C || !A || !X || !Q) return fail(W4A16_EARG, "null pointer");
    if (epilogue == W4A16_FUSED_ADD && !R) return fail(W4A16_EARG, "fused add needs a residual");
    if (!aligned16(A) || !aligned16(X) || (reinterpret_cast<uintptr_t>(C) & 3u) ||
        (reinterpret_cast<uintptr_t>(Q) & 3u) || (R && (reinterpret_cast<uintptr_t>(R) & 3u)))
        return fail(W4A16_EARG, "misaligned pointer (A and X need 16 bytes, C, Q, R need 4)");
    if (k == 0 || k % 128 != 0 || n_out % 16 != 0) return fail(W4A16_ESHAPE, "no feasible kernel found");
    return 0;
}

// The MFMA prefill kernels store (and read the residual) four features at a time.
int check_prefill_alignment(int algo_id, const void* C, const void* R, int epilogue)
{
    if (algo_at(algo_id).kind != 1 || epilogue == W4A16_FUSED_SILU_FFN) return 0;
    if (!aligned8(C) || (R && !aligned8(R)))
        return fail(W4A16_EARG, "misaligned pointer (C and R need 8 bytes for more than 32 tokens)");
    return 0;
}

// A handle's scratch, counters and events live on the device that was current at w4a16_create; a launch
// made with another device current would hand them to a GPU that cannot reach them.
int check_device(const w4a16_handle* h)
{
    int              dev = -1;
    const hipError_t e   = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev != h->device)
        return fail(W4A16_EARG, "the handle belongs to device %d but device %d is current", h->device, dev);
    return W4A16_OK;
}

// the kernel w4a16_gemm uses for algo_id < 0: a measured one if this exact shape was measured
int pick_for(const w4a16_handle* h, int n_out, int tokens, int k)
{
    const auto it = h->tuned.find(std::make_tuple(n_out, tokens, k));
    if (it != h->tuned.end() && algo_feasible(it->second, n_out, tokens, k, h->scratch)) return it->second;
    return algo_pick(n_out, tokens, k, h->scratch);
}

// The partial-tile workspace of a handle is allocated when a launch first needs it.  That cannot
// happen while `st` is being captured into a graph; `*have` then stays false.
int ensure_workspace(w4a16_handle* h, hipStream_t st, bool* have)
{
    *have = h->scratch.ws != nullptr;
    if (*have) return W4A16_OK;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) return W4A16_OK;
    const hipError_t e = hipMalloc((void**)&h->scratch.ws, kWorkspaceBytes);
    if (e != hipSuccess) {
        h->scratch.ws = nullptr;
        return hip_fail(e, "w4a16: allocating the split-K workspace");
    }
    *have = true;
    return W4A16_OK;
}

// what an algo may use of a scratch that has no workspace yet: nothing
Scratch without_workspace(const Scratch& sc)
{
    Scratch s = sc;
    s.ws       = nullptr;
    s.ws_bytes = 0;
    return s;
}

}  // namespace

extern "C" {

int w4a16_create(w4a16_handle** out)
{
    if (!out) return fail(W4A16_EARG, "null output pointer");
    *out = nullptr;
    auto*      h = new w4a16_handle();
    hipError_t e = hipGetDevice(&h->device);
    if (e == hipSuccess) e = hipEventCreate(&h->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&h->ev_end);
    if (e == hipSuccess) e = hipMalloc((void**)&h->scratch.cnt, kCounters * sizeof(int));
    if (e == hipSuccess) e = hipMemset(h->scratch.cnt, 0, kCounters * sizeof(int));
    if (e == hipSuccess) e = hipMalloc((void**)&h->sync, kSyncInts * sizeof(int));
    if (e == hipSuccess) e = hipMemset(h->sync, 0, kSyncInts * sizeof(int));
    if (e == hipSuccess) e = hipMalloc((void**)&h->clk, 4 * sizeof(unsigned long long));
    if (e == hipSuccess) e = hipMemset(h->clk, 0, 4 * sizeof(unsigned long long));
    if (e == hipSuccess) e = hipDeviceGetAttribute(&h->cus, hipDeviceAttributeMultiprocessorCount, h->device);
    int khz = 0;
    if (e == hipSuccess) e = hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, h->device);
    h->clock_khz  = khz > 0 ? khz : 100000;
    h->spin_ticks = 50 * h->clock_khz;  // 50 ms: a serving loop must not stall for longer than that
    if (e == hipSuccess) e = hipDeviceSynchronize();
    // a library set-up call on this device: also the moment to look up the static scratch array's address
    Scratch st{};
    if (e == hipSuccess) e = static_scratch(&st);
    if (e != hipSuccess) {
        if (h->ev_start) (void)hipEventDestroy(h->ev_start);
        if (h->ev_end) (void)hipEventDestroy(h->ev_end);
        if (h->scratch.cnt) (void)hipFree(h->scratch.cnt);
        if (h->sync) (void)hipFree(h->sync);
        if (h->clk) (void)hipFree(h->clk);
        delete h;
        return hip_fail(e, "w4a16_create");
    }
    h->scratch.ws       = nullptr;  // 64 MiB, allocated by the first launch that splits K (ensure_workspace)
    h->scratch.ws_bytes = kWorkspaceBytes;
    h->scratch.cnt_len  = kCounters;
    *out = h;
    return W4A16_OK;
}

void w4a16_destroy(w4a16_handle* h)
{
    if (!h) return;
    (void)hipEventDestroy(h->ev_end);
    (void)hipEventDestroy(h->ev_start);
    if (h->scratch.ws) (void)hipFree(h->scratch.ws);
    (void)hipFree(h->scratch.cnt);
    (void)hipFree(h->sync);
    (void)hipFree(h->clk);
    delete h;
}

int w4a16_pick(const w4a16_handle* h, int n_out, int tokens, int k)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (n_out <= 0 || tokens <= 0 || k <= 0 || k % 128 != 0 || n_out % 16 != 0)
        return fail(W4A16_ESHAPE, "no feasible kernel found");
    const int id = pick_for(h, n_out, tokens, k);
    return id >= 0 ? id : fail(W4A16_ESHAPE, "no feasible kernel found");
}

int w4a16_clear_tuning(w4a16_handle* h)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    h->tuned.clear();
    return W4A16_OK;
}

// File format: a header line that names the library version, the CU count of the device and the size of the kernel
// table - a measurement is only worth anything for that combination - then one line "n_out tokens k algo_id" per shape.
int w4a16_save_tuning(const w4a16_handle* h, const char* path)
{
    if (!h || !path) return fail(W4A16_EARG, "save_tuning: null argument");
    FILE* f = fopen(path, "w");
    if (!f) return fail(W4A16_EARG, "save_tuning: cannot open %s for writing", path);
    fprintf(f, "w4a16-tuning 1 \"%s\" cus=%d algos=%d\n", w4a16_version(), h->cus, algo_count());
    for (const auto& kv : h->tuned)
        fprintf(f, "%d %d %d %d\n", std::get<0>(kv.first), std::get<1>(kv.first), std::get<2>(kv.first), kv.second);
    const bool bad = ferror(f) != 0;
    if (fclose(f) != 0 || bad) return fail(W4A16_EARG, "save_tuning: writing %s failed", path);
    return (int)h->tuned.size();
}

int w4a16_load_tuning(w4a16_handle* h, const char* path)
{
    if (!h || !path) return fail(W4A16_EARG, "load_tuning: null argument");
    FILE* f = fopen(path, "r");
    if (!f) return fail(W4A16_EARG, "load_tuning: cannot open %s", path);
    char version[128] = "";
    int  cus = 0, algos = 0, fmt = 0;
    const int got = fscanf(f, "w4a16-tuning %d \"%127[^\"]\" cus=%d algos=%d", &fmt, version, &cus, &algos);
    if (got != 4 || fmt != 1) {
        fclose(f);
        return fail(W4A16_EARG, "load_tuning: %s is not a tuning file", path);
    }
    if (strcmp(version, w4a16_version()) != 0 || cus != h->cus || algos != algo_count()) {
        fclose(f);
        return fail(W4A16_ETUNING, "load_tuning: %s was measured with \"%s\" on %d CUs (%d kernels); this is \"%s\" on %d CUs "
                                   "(%d kernels): ignored", path, version, cus, algos, w4a16_version(), h->cus, algo_count());
    }
    int n_out, tokens, k, id, loaded = 0;
    while (fscanf(f, "%d %d %d %d", &n_out, &tokens, &k, &id) == 4) {
        if (n_out <= 0 || tokens <= 0 || k <= 0 || id < 0 || id >= algo_count()) continue;
        if (!algo_feasible(id, n_out, tokens, k, h->scratch)) continue;
        h->tuned[std::make_tuple(n_out, tokens, k)] = id;
        ++loaded;
    }
    fclose(f);
    return loaded;
}

int w4a16_algo_count(void)
{
    return algo_count();
}

// What w4a16_gemm decides before it launches: the kernel and the scratch it may use.  Everything that can
// fail for reasons other than the launch itself happens here, so that a list of GEMMs can be planned as a
// whole before the first of them is enqueued.
struct GemmPlan {
    int     algo;
    Scratch sc;
    int     nq;  // quantisation groups per 128-row weight tile: 1 = the kernel table, 2 or 4 = the kernel for group size 64 / 32
};

// Group sizes 64 and 32 have two kernels outside the table (strips for few tokens, one MFMA tile for many): chosen
// by rule, no scratch.
constexpr int kGroupsStrips = -1, kGroupsMfma = -2;
int plan_small_groups(const void* C, const void* R, int n_out, int tokens, int k, int group_size, int epilogue, int algo_id,
                      GemmPlan* out)
{
    if (algo_id >= 0)
        return fail(W4A16_EALGO, "kernel ids belong to group size 128; group size %d takes algo_id < 0 only", group_size);
    const int nq = 128 / group_size;
    if (!strip_groups_feasible(nq, n_out, tokens, k)) return fail(W4A16_ESHAPE, "no feasible kernel found");
    out->algo = kGroupsStrips;
    out->sc   = Scratch{};
    out->nq   = nq;
    // Many tokens: the 256 x 128 MFMA tile (n_out a multiple of 128) once its K steps cost less than streaming the
    // weights once per 16 tokens.  Step and stream figures measured on Llama-2-7B shapes with group size 64.
    if (prefill_groups_feasible(nq, n_out, tokens, k)) {
        const double tiles    = (double)((tokens + 255) / 256) * (n_out / 128);
        const double mfma_us  = 3.0 + std::ceil(tiles / 256.0) * (k / 128) * 2.4;
        const double strip_us = (double)((tokens + 15) / 16) * (3.0 + ((double)k * n_out / 2) / 3.0e6);
        // (the MFMA kernel stores four features at a time: a pointer it cannot take leaves the GEMM with the strips)
        const bool aligned = epilogue == W4A16_FUSED_SILU_FFN || (aligned8(C) && (!R || aligned8(R)));
        if (mfma_us < strip_us && aligned) out->algo = kGroupsMfma;
    }
    return W4A16_OK;
}

hipError_t launch_plan(const GemmPlan& plan, const GemmArgs& g, hipStream_t st)
{
    if (plan.nq > 1) return plan.algo == kGroupsMfma ? prefill_groups_launch(plan.nq, g, st) : strip_groups_launch(plan.nq, g, st);
    return algo_launch(plan.algo, g, plan.sc, st);
}

int plan_gemm(w4a16_handle* h, const void* C, const void* R, int n_out, int tokens, int k, int group_size, int epilogue,
              int algo_id, hipStream_t st, GemmPlan* out)
{
    if (group_size != 128) return plan_small_groups(C, R, n_out, tokens, k, group_size, epilogue, algo_id, out);
    out->nq = 1;
    if (algo_id >= algo_count()) return fail(W4A16_EALGO, "algo_id %d out of range (0..%d)", algo_id, algo_count() - 1);
    const bool chosen = algo_id >= 0;
    if (!chosen) algo_id = pick_for(h, n_out, tokens, k);
    if (algo_id < 0 || !algo_feasible(algo_id, n_out, tokens, k, h->scratch))
        return fail(W4A16_ESHAPE, "no feasible kernel found");
    Scratch sc = h->scratch;
    if (algo_scratch_bytes(algo_id, n_out, tokens, k, sc) > 0) {
        bool have = false;
        if (int rc = ensure_workspace(h, st, &have)) return rc;
        sc = h->scratch;
        if (!have) {
            // the stream is being captured and this handle has never split K before: nothing can be allocated now
            sc = without_workspace(sc);
            if (!chosen) algo_id = algo_pick(n_out, tokens, k, sc);
            if (algo_id < 0 || !algo_feasible(algo_id, n_out, tokens, k, sc))
                return fail(W4A16_ESCRATCH, "this kernel splits K through the handle's workspace, which cannot be "
                                            "allocated while the stream is capturing: run the shape once before");
        }
    }
    if (int rc = check_prefill_alignment(algo_id, C, R, epilogue)) return rc;
    out->algo = algo_id;
    out->sc   = sc;
    return W4A16_OK;
}

int w4a16_gemm(w4a16_handle* h, void* C, const void* A, const void* X, const void* Q, const void* R, int n_out,
               int tokens, int k, int group_size, int epilogue, int algo_id, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    const int chk = check_gemm_args(C, A, X, Q, R, n_out, tokens, k, group_size, epilogue);
    if (chk < 0) return chk;
    if (chk > 0) return W4A16_OK;
    if (algo_id >= algo_count()) return fail(W4A16_EALGO, "algo_id %d out of range (0..%d)", algo_id, algo_count() - 1);
    if (int rc = check_device(h)) return rc;
    GemmPlan plan{};
    if (int rc = plan_gemm(h, C, R, n_out, tokens, k, group_size, epilogue, algo_id, (hipStream_t)stream, &plan)) return rc;
    GemmArgs g{(uint16_t*)C, (const uint32_t*)A, (const uint16_t*)X, (const uint32_t*)Q, (const uint16_t*)R,
               n_out,        tokens,             k,                  epilogue};
    if (h->clk_on) g.clk = h->clk;
    const hipError_t e = launch_plan(plan, g, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "w4a16_gemm launch");
    return W4A16_OK;
}

int w4a16_gemm_static(void* C, const void* A, const void* X, const void* Q, const void* R, int n_out, int tokens,
                      int k, int group_size, int epilogue, int algo_id, void* stream)
{
    const int chk = check_gemm_args(C, A, X, Q, R, n_out, tokens, k, group_size, epilogue);
    if (chk < 0) return chk;
    if (chk > 0) return W4A16_OK;
    if (algo_id >= algo_count()) return fail(W4A16_EALGO, "algo_id %d out of range (0..%d)", algo_id, algo_count() - 1);
    if (group_size != 128) {  // one kernel, no scratch at all
        GemmPlan plan{};
        if (int rc = plan_small_groups(C, R, n_out, tokens, k, group_size, epilogue, algo_id, &plan)) return rc;
        GemmArgs g{(uint16_t*)C, (const uint32_t*)A, (const uint16_t*)X, (const uint32_t*)Q, (const uint16_t*)R,
                   n_out,        tokens,             k,                  epilogue};
        const hipError_t e = launch_plan(plan, g, (hipStream_t)stream);
        return e == hipSuccess ? W4A16_OK : hip_fail(e, "w4a16_gemm_static launch");
    }
    Scratch sc{};
    if (const hipError_t e = static_scratch(&sc); e != hipSuccess) return hip_fail(e, "w4a16_gemm_static set-up");
    if (algo_id < 0) algo_id = algo_pick(n_out, tokens, k, sc);
    if (algo_id < 0) return fail(W4A16_ESHAPE, "no feasible kernel found");
    if (!algo_feasible(algo_id, n_out, tokens, k, sc)) {
        // feasible with a handle's (larger) workspace?  Then it is the static buffer that is too small.
        Scratch big{nullptr, kWorkspaceBytes, nullptr, kCounters};
        if (algo_feasible(algo_id, n_out, tokens, k, big))
            return fail(W4A16_ESCRATCH, "algo %d needs %zu bytes of split-K scratch for this shape; the static buffer holds %zu "
                                        "bytes and %d counters",
                        algo_id, algo_scratch_bytes(algo_id, n_out, tokens, k, big), sc.ws_bytes, sc.cnt_len);
        return fail(W4A16_ESHAPE, "no feasible kernel found");
    }
    if (int rc = check_prefill_alignment(algo_id, C, R, epilogue)) return rc;
    const hipStream_t st = (hipStream_t)stream;
    if (algo_scratch_bytes(algo_id, n_out, tokens, k, sc) > 0) {
        // every call on this GPU shares the array, whatever an earlier (perhaps aborted) call left in it
        // (only the counters this launch will use: one per output tile or column block, never more than workgroups)
        const int used = std::min(sc.cnt_len, algo_grid(algo_id, n_out, tokens, k, sc));
        if (const hipError_t e = clear_counters(sc, used, st); e != hipSuccess) return hip_fail(e, "w4a16_gemm_static clear");
    }
    GemmArgs g{(uint16_t*)C, (const uint32_t*)A, (const uint16_t*)X, (const uint32_t*)Q, (const uint16_t*)R,
               n_out,        tokens,             k,                  epilogue};
    const hipError_t e = algo_launch(algo_id, g, sc, st);
    if (e != hipSuccess) return hip_fail(e, "w4a16_gemm_static launch");
    return W4A16_OK;
}

int w4a16_gemm_sequence(w4a16_handle* h, const w4a16_gemm_desc* gemms, int count, int tokens, int group_size,
                        int flags, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (count < 0 || (count > 0 && !gemms)) return fail(W4A16_EARG, "bad sequence");
    if (flags & ~W4A16_SEQ_PERSISTENT) return fail(W4A16_EARG, "unknown sequence flags %d", flags);
    // validate everything before anything is launched
    for (int i = 0; i < count; ++i) {
        const w4a16_gemm_desc& d = gemms[i];
        const int chk = check_gemm_args(d.C, d.A, d.X, d.Q, d.R, d.n_out, tokens, d.k, group_size, d.epilogue);
        if (chk < 0) return chk;
        if (chk > 0 && tokens != 0) return fail(W4A16_EARG, "GEMM %d of the sequence is empty", i);
    }
    if (tokens == 0 || count == 0) return W4A16_OK;
    if (int rc = check_device(h)) return rc;
    if (!(flags & W4A16_SEQ_PERSISTENT) || tokens > 16 || count == 1 || group_size != 128) {
        // One launch per GEMM; stream order gives the dependencies.  Every GEMM is planned (kernel, workspace,
        // alignment) before the first one is launched: a list that cannot run as a whole runs not at all.
        std::vector<GemmPlan> plans(count);
        for (int i = 0; i < count; ++i) {
            const w4a16_gemm_desc& d = gemms[i];
            if (int rc = plan_gemm(h, d.C, d.R, d.n_out, tokens, d.k, group_size, d.epilogue, -1, (hipStream_t)stream, &plans[i]))
                return rc;
        }
        for (int i = 0; i < count; ++i) {
            const w4a16_gemm_desc& d = gemms[i];
            GemmArgs g{(uint16_t*)d.C, (const uint32_t*)d.A, (const uint16_t*)d.X, (const uint32_t*)d.Q, (const uint16_t*)d.R,
                       d.n_out,        tokens,                d.k,                  d.epilogue};
            const hipError_t e = launch_plan(plans[i], g, (hipStream_t)stream);
            if (e != hipSuccess) return hip_fail(e, "w4a16_gemm_sequence launch");  // (the launch itself: earlier GEMMs are enqueued)
        }
        return W4A16_OK;
    }
    SeqGemm chunk[kSeqMax];
    for (int first = 0; first < count; first += kSeqMax) {
        const int n = std::min(kSeqMax, count - first);
        for (int i = 0; i < n; ++i) {
            const w4a16_gemm_desc& d = gemms[first + i];
            chunk[i] = SeqGemm{(uint16_t*)d.C, (const u32x4_t*)d.A, (const uint16_t*)d.X, (const uint32_t*)d.Q,
                               (const uint16_t*)d.R, d.n_out, d.k, d.epilogue, (i > 0 && d.depends) ? 1 : 0};
        }
        if (!sequence_feasible(chunk, n, tokens)) return fail(W4A16_ESHAPE, "no feasible kernel found");
        const hipError_t e = sequence_launch(chunk, n, tokens, h->sync, h->cus, h->spin_ticks, (hipStream_t)stream);
        if (e != hipSuccess) return hip_fail(e, "w4a16_gemm_sequence launch");
    }
    return W4A16_OK;
}

int w4a16_sequence_status(w4a16_handle* h, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (int rc = check_device(h)) return rc;
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "w4a16_sequence_status");
    int word = 0;
    e = hipMemcpy(&word, h->sync + sequence_error_index(), sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "w4a16_sequence_status");
    if (word == 0) return W4A16_OK;
    // the launch that gave up may have left counters behind; cleared in stream order, then waited for
    e = hipMemsetAsync(h->sync, 0, kSyncInts * sizeof(int), (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "w4a16_sequence_status");
    return fail(W4A16_ETIMEOUT, "a workgroup of w4a16_gemm_sequence gave up waiting at a device-wide barrier: the "
                                "grid was not resident all at once; the outputs of that launch are undefined");
}

int w4a16_set_barrier_timeout(w4a16_handle* h, double seconds)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (!(seconds >= 0.0) || seconds > 3600.0) return fail(W4A16_EARG, "timeout out of range");
    h->spin_ticks = (long long)(seconds * 1000.0 * (double)h->clock_khz);
    return W4A16_OK;
}

int w4a16_ffn(w4a16_handle* h, void* ffn_output, void* gating_buf, const void* ffn_input, const void* A13,
              const void* Q13, const void* A2, const void* Q2, const void* residual, int hidden_units,
              int inter_size, int tokens, int group_size, void* stream)
{
    if (hidden_units < 0 || inter_size < 0) return fail(W4A16_EARG, "negative size");
    const w4a16_gemm_desc seq[2] = {
        {gating_buf, A13, ffn_input, Q13, nullptr, 2 * inter_size, hidden_units, W4A16_FUSED_SILU_FFN, 0},
        {ffn_output, A2, gating_buf, Q2, residual, hidden_units, inter_size, residual ? W4A16_FUSED_ADD : W4A16_GEMM, 1}};
    return w4a16_gemm_sequence(h, seq, 2, tokens, group_size, 0, stream);
}

int w4a16_measure(w4a16_handle* h, void* C, const void* A, const void* X, const void* Q, const void* R, int n_out,
                  int tokens, int k, int group_size, int epilogue, w4a16_metric* metrics, int capacity, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    const int chk = check_gemm_args(C, A, X, Q, R, n_out, tokens, k, group_size, epilogue);
    if (chk < 0) return chk;
    if (group_size != 128) return fail(W4A16_EGROUP, "unsupported group size");  // (64 and 32 have one kernel: nothing to measure)
    if (!metrics || capacity <= 0) return fail(W4A16_EARG, "no room for metrics");
    if (chk > 0) return 0;
    if (int rc = check_device(h)) return rc;
    constexpr int kWarmup = 10, kMeasure = 100;  // gemm_s4_f16.cu:258-259
    hipStream_t   st   = (hipStream_t)stream;
    bool          have = false;
    if (int rc = ensure_workspace(h, st, &have)) return rc;
    if (!have) return fail(W4A16_EARG, "w4a16_measure synchronises: it cannot run on a capturing stream");
    if (!aligned8(C) || (R && !aligned8(R))) return fail(W4A16_EARG, "misaligned pointer (w4a16_measure needs C and R aligned to 8 bytes)");
    const int     best = pick_for(h, n_out, tokens, k);
    GemmArgs g{(uint16_t*)C, (const uint32_t*)A, (const uint16_t*)X, (const uint32_t*)Q, (const uint16_t*)R,
               n_out,        tokens,             k,                  epilogue};
    std::vector<w4a16_metric> all;
    for (int id = 0; id < algo_count(); ++id) {
        const Algo&  a = algo_at(id);
        w4a16_metric m{};
        m.id       = id;
        m.kind     = a.kind;
        m.tile_n   = a.kind == 2 ? 16 * strip_width(a.param, a.tile_t, n_out, tokens, k) : a.tile_n;
        m.tile_t   = a.tile_t;
        m.slices   = a.slices;
        m.best     = id == best;
        m.feasible = algo_feasible(id, n_out, tokens, k, h->scratch);
        m.count    = 1;
        m.ms       = std::numeric_limits<float>::infinity();
        if (m.feasible) {
            m.grid = algo_grid(id, n_out, tokens, k, h->scratch);
            for (int j = 0; j < kWarmup + kMeasure; ++j) {
                if (j == kWarmup) (void)hipEventRecord(h->ev_start, st);
                const hipError_t e = algo_launch(id, g, h->scratch, st);
                if (e != hipSuccess) return hip_fail(e, "w4a16_measure launch");
            }
            (void)hipEventRecord(h->ev_end, st);
            hipError_t e = hipEventSynchronize(h->ev_end);
            if (e != hipSuccess) return hip_fail(e, "w4a16_measure sync");
            float ms = 0.f;
            e        = hipEventElapsedTime(&ms, h->ev_start, h->ev_end);
            if (e != hipSuccess) return hip_fail(e, "w4a16_measure elapsed");
            m.ms    = ms;
            m.count = kMeasure;
        }
        all.push_back(m);
    }
    std::stable_sort(all.begin(), all.end(), [](const w4a16_metric& a, const w4a16_metric& b) { return a.ms < b.ms; });
    if (!all.empty() && all.front().feasible) h->tuned[std::make_tuple(n_out, tokens, k)] = all.front().id;
    const int n = std::min<int>(capacity, (int)all.size());
    std::memcpy(metrics, all.data(), sizeof(w4a16_metric) * n);
    return n;
}

static int check_repack(const char* what, int m, int k, int m_mult, int k_mult)
{
    if (m < 0 || k < 0) return fail(W4A16_EARG, "%s: negative size", what);
    if (m % m_mult != 0 || k % k_mult != 0)
        return fail(W4A16_ESHAPE, "%s: m must be a multiple of %d and k of %d (got m=%d k=%d)", what, m_mult, k_mult, m, k);
    return 0;
}

int w4a16_convert_s4_k_m8(uint32_t* A_dst, void* Q_dst, void* workspace, const uint32_t* A_src, const void* scales,
                          const uint32_t* qzeros, int m, int k, int group_size, void* stream)
{
    (void)workspace;
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (int c = check_repack("convert_s4_k_m8", m, k, 16, 128)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if (!A_dst || !Q_dst || !A_src || !scales || !qzeros) return fail(W4A16_EARG, "convert_s4_k_m8: null pointer");
    const hipError_t e = launch_convert(A_dst, (uint32_t*)Q_dst, A_src, (const uint16_t*)scales, qzeros, m, k,
                                        group_size, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "convert_s4_k_m8");
}

int w4a16_deploy_qkv(uint32_t* A_dst, void* Q_dst, const uint32_t* const qweight[3], const uint32_t* const qzeros[3],
                     const void* const scales[3], int n_q, int n_kv, int k, int size_per_head, int group_size, void* stream)
{
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (n_q < 0 || n_kv < 0 || k < 0) return fail(W4A16_EARG, "deploy_qkv: negative size");
    if (size_per_head <= 0 || size_per_head % 2 != 0 || n_q % size_per_head != 0 || n_kv % size_per_head != 0)
        return fail(W4A16_ESHAPE, "deploy_qkv: q and k widths must be multiples of an even size_per_head");
    if (n_q % 8 != 0 || n_kv % 8 != 0) return fail(W4A16_ESHAPE, "deploy_qkv: widths must be multiples of 8");
    if (int c = check_repack("deploy_qkv", n_q + 2 * n_kv, k, 16, 128)) return c;
    if (n_q + 2 * n_kv == 0 || k == 0) return W4A16_OK;
    if (!A_dst || !Q_dst || !qweight || !qzeros || !scales) return fail(W4A16_EARG, "deploy_qkv: null pointer");
    const int       width[3]  = {n_q, n_kv, n_kv};
    const int       rotary[3] = {size_per_head, size_per_head, 0};
    const uint16_t* s[3];
    for (int i = 0; i < 3; ++i) {
        if (width[i] > 0 && (!qweight[i] || !qzeros[i] || !scales[i])) return fail(W4A16_EARG, "deploy_qkv: null pointer");
        s[i] = (const uint16_t*)scales[i];
    }
    const hipError_t e = launch_deploy(A_dst, (uint32_t*)Q_dst, qweight, qzeros, s, width, rotary, 0, k, group_size, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "deploy_qkv");
}

int w4a16_deploy_w13(uint32_t* A_dst, void* Q_dst, const uint32_t* w1_qweight, const uint32_t* w3_qweight,
                     const uint32_t* w1_qzeros, const uint32_t* w3_qzeros, const void* w1_scales, const void* w3_scales,
                     int inter_size, int k, int group_size, void* stream)
{
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (inter_size < 0 || k < 0) return fail(W4A16_EARG, "deploy_w13: negative size");
    if (int c = check_repack("deploy_w13", inter_size, k, 8, 128)) return c;
    if (inter_size == 0 || k == 0) return W4A16_OK;
    if (!A_dst || !Q_dst || !w1_qweight || !w3_qweight || !w1_qzeros || !w3_qzeros || !w1_scales || !w3_scales)
        return fail(W4A16_EARG, "deploy_w13: null pointer");
    const uint32_t* qw[3]     = {w1_qweight, w3_qweight, nullptr};
    const uint32_t* qz[3]     = {w1_qzeros, w3_qzeros, nullptr};
    const uint16_t* s[3]      = {(const uint16_t*)w1_scales, (const uint16_t*)w3_scales, nullptr};
    const int       width[3]  = {inter_size, inter_size, 0};
    const int       rotary[3] = {0, 0, 0};
    const hipError_t e = launch_deploy(A_dst, (uint32_t*)Q_dst, qw, qz, s, width, rotary, 1, k, group_size, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "deploy_w13");
}

int w4a16_reformat_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, void* stream)
{
    if (int c = check_repack("reformat_s4_k_m8", m, k, 16, 128)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if (!dst || !src) return fail(W4A16_EARG, "reformat_s4_k_m8: null pointer");
    const hipError_t e = launch_convert(dst, nullptr, src, nullptr, nullptr, m, k, 128, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "reformat_s4_k_m8");
}

int w4a16_fuse_w1_w3_s4_k_m8(uint32_t* dst, const uint32_t* src, int m, int k, void* stream)
{
    if (int c = check_repack("fuse_w1_w3_s4_k_m8", m, k, 8, 1)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if (!dst || !src) return fail(W4A16_EARG, "fuse_w1_w3_s4_k_m8: null pointer");
    const hipError_t e = launch_fuse_w1_w3(dst, src, m, k, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "fuse_w1_w3_s4_k_m8");
}

int w4a16_transpose_qk_s4_k_m8_hf(uint32_t* dst, const uint32_t* src, int m, int k, int size_per_head, void* stream)
{
    if (size_per_head <= 0 || size_per_head % 2 != 0) return fail(W4A16_ESHAPE, "transpose_qk: bad size_per_head");
    if (int c = check_repack("transpose_qk_s4_k_m8_hf", m, k, 8, 1)) return c;
    if (m % size_per_head != 0) return fail(W4A16_ESHAPE, "transpose_qk: m is not a multiple of size_per_head");
    if (m == 0 || k == 0) return W4A16_OK;
    if (!dst || !src) return fail(W4A16_EARG, "transpose_qk_s4_k_m8_hf: null pointer");
    const hipError_t e = launch_transpose_qk(dst, src, m, k, size_per_head, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "transpose_qk_s4_k_m8_hf");
}

int w4a16_dequantize_s4(void* dst, const uint32_t* src, size_t count, void* stream)
{
    if (count == 0) return W4A16_OK;
    if (!dst || !src) return fail(W4A16_EARG, "dequantize_s4: null pointer");
    if (!aligned16(dst)) return fail(W4A16_EARG, "dequantize_s4: dst needs 16-byte alignment");
    const hipError_t e = launch_dequantize_s4(dst, src, count, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "dequantize_s4");
}

int w4a16_unpack_repacked(uint32_t* qweight, uint32_t* qzeros, void* scales, const uint32_t* A, const void* Q, int m,
                          int k, int group_size, void* stream)
{
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (int c = check_repack("unpack_repacked", m, k, 16, 128)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if ((qweight && !A) || ((qzeros || scales) && !Q)) return fail(W4A16_EARG, "unpack_repacked: null pointer");
    const hipError_t e = launch_unpack(qweight, qzeros, (uint16_t*)scales, A, (const uint32_t*)Q, m, k,
                                       group_size, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "unpack_repacked");
}

int w4a16_dequantize_repacked(void* W, const uint32_t* A, const void* Q, int m, int k, int group_size, void* stream)
{
    if (!group_ok(group_size)) return fail(W4A16_EGROUP, "unsupported group size");
    if (int c = check_repack("dequantize_repacked", m, k, 16, 128)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if (!W || !A || !Q) return fail(W4A16_EARG, "dequantize_repacked: null pointer");
    const hipError_t e = launch_dequantize_repacked((uint16_t*)W, A, (const uint32_t*)Q, m, k, group_size, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "dequantize_repacked");
}

int w4a16_from_reference_layout(uint32_t* A_dst, const uint32_t* A_ref, int m, int k, void* stream)
{
    if (int c = check_repack("from_reference_layout", m, k, 32, 128)) return c;
    if (m == 0 || k == 0) return W4A16_OK;
    if (!A_dst || !A_ref) return fail(W4A16_EARG, "from_reference_layout: null pointer");
    const hipError_t e = launch_from_reference(A_dst, A_ref, m, k, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "from_reference_layout");
}

int w4a16_probe_read(w4a16_handle* h, const void* src, size_t bytes, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (!src || !aligned16(src)) return fail(W4A16_EARG, "probe_read: src must be a 16-byte aligned device pointer");
    // the sink (one word per workgroup, practically never written) is the unused tail of the barrier area
    static_assert(kSyncInts - 64 * 40 >= 8 * 256, "no room for the probe's sink");
    if (h->cus > 256) return fail(W4A16_ESHAPE, "probe_read: more than 256 CUs");
    if (int rc = check_device(h)) return rc;
    const hipError_t e = launch_probe_read(src, bytes, h->sync + 64 * 40, h->cus, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "probe_read");
}

int w4a16_probe_stream(w4a16_handle* h, const void* src, size_t bytes, int wg_per_cu, int in_flight, int hint, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (!src || !aligned16(src)) return fail(W4A16_EARG, "probe_stream: src must be a 16-byte aligned device pointer");
    if (!probe_stream_config_ok(wg_per_cu, in_flight, hint))
        return fail(W4A16_EARG, "probe_stream: wg_per_cu is 1, 2 or 4, in_flight 2, 4, 8 or 16, hint 0, 1 or 2");
    if (h->cus > 256) return fail(W4A16_ESHAPE, "probe_stream: more than 256 CUs");
    if (int rc = check_device(h)) return rc;
    const hipError_t e = launch_probe_stream(src, bytes, h->sync + 64 * 40, h->cus, wg_per_cu, in_flight, hint, (hipStream_t)stream,
                                             h->clk_on ? h->clk : nullptr);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "probe_stream");
}

int w4a16_probe_mfma(w4a16_handle* h, int waves_per_cu, int iters, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (waves_per_cu != 4 && waves_per_cu != 8 && waves_per_cu != 16) return fail(W4A16_EARG, "probe_mfma: waves_per_cu is 4, 8 or 16");
    if (iters < 1 || iters > (1 << 24)) return fail(W4A16_EARG, "probe_mfma: iters out of range");
    if (int rc = check_device(h)) return rc;
    const hipError_t e = launch_probe_mfma(h->sync + 64 * 40, h->cus, waves_per_cu, iters, h->clk_on ? h->clk : nullptr, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "probe_mfma");
}

int w4a16_probe_clock_begin(w4a16_handle* h, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (int rc = check_device(h)) return rc;
    const hipError_t e = hipMemsetAsync(h->clk, 0, 4 * sizeof(unsigned long long), (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "probe_clock_begin");
    h->clk_on = true;
    return W4A16_OK;
}

int w4a16_probe_clock_end(w4a16_handle* h, unsigned long long* cycles, unsigned long long* ticks, unsigned long long* launches,
                          long long* ticks_per_second, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (!cycles || !ticks || !launches) return fail(W4A16_EARG, "probe_clock_end: null output pointer");
    if (int rc = check_device(h)) return rc;
    h->clk_on = false;
    unsigned long long v[4] = {0, 0, 0, 0};
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e == hipSuccess) e = hipMemcpy(v, h->clk, sizeof(v), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "probe_clock_end");
    *cycles = v[0], *ticks = v[1], *launches = v[2];
    if (ticks_per_second) *ticks_per_second = h->clock_khz * 1000;
    return W4A16_OK;
}

int w4a16_probe_barrier(w4a16_handle* h, int iters, int tree, void* stream)
{
    if (!h) return fail(W4A16_EARG, "null handle");
    if (iters < 1 || iters > (1 << 20)) return fail(W4A16_EARG, "probe_barrier: iters out of range");
    if (int rc = check_device(h)) return rc;
    const hipError_t e = launch_probe_barrier(h->sync, iters, tree, h->cus, h->spin_ticks, (hipStream_t)stream);
    return e == hipSuccess ? W4A16_OK : hip_fail(e, "probe_barrier");
}

const char* w4a16_last_error(void)
{
    return g_err;
}

const char* w4a16_version(void)
{
    return "w4a16-gfx950 0.3";
}

}  // extern "C"
