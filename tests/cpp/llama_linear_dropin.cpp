// The drop-in boundary, exercised the way the engine does: a LlamaLinear-shaped caller written
// against the reference's interface (src/turbomind/models/llama/LlamaLinear.h:15-87 in lmdeploy)
// using only the names the reference uses.  It links the system HIP runtime, converts a small
// AWQ matrix with convert_s4_k_m8 and runs the three epilogues on a case whose answer is known in
// closed form: q - z = 1 and s = 1 everywhere, every activation 1/16, K = 256, so every GEMM
// output is exactly 16; SiLU-gated pairs give fp16(16 / (1 + exp(-16)) * 16) = 256 and the residual
// epilogue 16 + 1 = 17.  Outputs are poisoned before each call.  On a machine without a GPU the
// constructor throws and the program says so instead.
#include "turbomind/format.h"
#include "turbomind/gemm_s4_f16.h"

#include <cstdio>
#include <cstring>
#include <sstream>
#include <type_traits>
#include <string>
#include <vector>

namespace turbomind {

using cudaStream_t = hipStream_t;  // the one line a HIP build of the engine adds
using uint         = unsigned int;

enum class WeightType : int { kFP32, kFP16, kFP8, kINT8, kINT4 };

template<typename T>
struct LlamaDenseWeight {  // LlamaDenseWeight.h:56-64
    size_t     input_dims;
    size_t     output_dims;
    void*      kernel;
    WeightType type;
    T*         bias;
    T*         scales_and_zeros;
    int        group_size;
};

template<typename T>
class LlamaLinear {
public:
    enum Type { kGemm, kFusedSiluFfn };
    explicit LlamaLinear(cudaStream_t stream): stream_(stream) {}

    void forward(T* output_data, const T* input_data, int batch_size, const LlamaDenseWeight<T>& weight, Type type = kGemm)
    {
        if constexpr (std::is_same_v<T, half>) {
            gemm_s4_f16_.Run(output_data,
                             (const uint*)weight.kernel,
                             input_data,
                             (const half2*)weight.scales_and_zeros,
                             weight.output_dims,
                             batch_size,
                             weight.input_dims,
                             weight.group_size,
                             type == kFusedSiluFfn ? GemmS4F16::kFusedSiluFfn : GemmS4F16::kGemm,
                             -1,
                             stream_);
        }
    }

private:
    cudaStream_t stream_{};
    GemmS4F16    gemm_s4_f16_;
};

}  // namespace turbomind

namespace {

template<typename T>
T* upload(const std::vector<T>& host)
{
    T* p = nullptr;
    if (hipMalloc((void**)&p, host.size() * sizeof(T)) != hipSuccess) throw std::runtime_error("hipMalloc");
    if (hipMemcpy(p, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess)
        throw std::runtime_error("hipMemcpy");
    return p;
}

// number of outputs that differ from the fp16 bit pattern `want`
int mismatches(const unsigned short* dev, size_t count, unsigned short want)
{
    std::vector<unsigned short> out(count);
    if (hipMemcpy(out.data(), dev, count * 2, hipMemcpyDeviceToHost) != hipSuccess) return -1;
    int bad = 0;
    for (auto v : out) bad += v != want;
    return bad;
}

}  // namespace

int main()
{
    using namespace turbomind;
    static_assert(GemmS4F16::kGemm == 0 && GemmS4F16::kFusedSiluFfn == 1 && GemmS4F16::kFusedAdd == 2, "enum values");
    try {
        hipStream_t stream = nullptr;
        if (hipStreamCreate(&stream) != hipSuccess) throw std::runtime_error("hipStreamCreate");
        LlamaLinear<half> linear(stream);
        const int         K = 256, N = 64, G = K / 128;
        constexpr unsigned short kOneSixteenth = 0x2c00, kOne = 0x3c00, k16 = 0x4c00, k17 = 0x4c40, k256 = 0x5c00,
                                 kPoison = 0x7e00;
        uint32_t* qw = upload(std::vector<uint32_t>(K * N / 8, 0x44444444u));  // q = 4
        uint32_t* qz = upload(std::vector<uint32_t>(G * N / 8, 0x33333333u));  // z = 3
        half*     s  = (half*)upload(std::vector<unsigned short>(G * N, kOne));
        uint32_t* A  = upload(std::vector<uint32_t>(K * N / 8, 0u));
        half2*    Q  = (half2*)upload(std::vector<uint32_t>(G * N, 0u));
        half*     ws = (half*)upload(std::vector<unsigned short>(G * N, 0));
        convert_s4_k_m8(A, Q, ws, qw, s, qz, N, K, 128, stream);
        LlamaDenseWeight<half> w{(size_t)K, (size_t)N, A, WeightType::kINT4, nullptr, (half*)Q, 128};

        int failed = 0;
        for (int T : {4, 100}) {  // a decode kernel and an MFMA prefill kernel
            half* X = (half*)upload(std::vector<unsigned short>((size_t)T * K, kOneSixteenth));
            half* R = (half*)upload(std::vector<unsigned short>((size_t)T * N, kOne));
            half* C = (half*)upload(std::vector<unsigned short>((size_t)T * N, kPoison));
            linear.forward(C, X, T, w);
            (void)hipStreamSynchronize(stream);
            const int bad_gemm = mismatches((const unsigned short*)C, (size_t)T * N, k16);

            (void)hipMemcpy(C, std::vector<unsigned short>((size_t)T * N, kPoison).data(), (size_t)T * N * 2,
                            hipMemcpyHostToDevice);
            linear.forward(C, X, T, w, LlamaLinear<half>::kFusedSiluFfn);
            (void)hipStreamSynchronize(stream);
            const int bad_silu = mismatches((const unsigned short*)C, (size_t)T * N / 2, k256);
            const int untouched = mismatches((const unsigned short*)C + (size_t)T * N / 2, (size_t)T * N / 2, kPoison);

            (void)hipMemcpy(C, std::vector<unsigned short>((size_t)T * N, kPoison).data(), (size_t)T * N * 2,
                            hipMemcpyHostToDevice);
            GemmS4F16 gemm;
            gemm.Run(C, A, X, Q, R, N, T, K, 128, GemmS4F16::kFusedAdd, -1, stream);
            (void)hipStreamSynchronize(stream);
            const int bad_add = mismatches((const unsigned short*)C, (size_t)T * N, k17);

            std::printf("drop-in GEMM ran, tokens %d: kGemm mismatches %d, kFusedSiluFfn mismatches %d (+%d written past the "
                        "output), kFusedAdd mismatches %d\n",
                        T, bad_gemm, bad_silu, untouched, bad_add);
            failed += (bad_gemm != 0) + (bad_silu != 0) + (untouched != 0) + (bad_add != 0);
            if (T == 4) {  // Measure with the dump flag set prints one table and clears the flag (gemm_s4_f16.cu:160-163)
                std::vector<Metric> metrics;
                std::ostringstream  table;
                gemm.Measure(C, A, X, Q, N, T, K, 128, GemmS4F16::kGemm, metrics, stream);
                DumpMetrics(table, metrics);
                const bool ok = !metrics.empty() && metrics.front().feasible && table.str().find("time_us") != std::string::npos;
                std::printf("Measure returned %zu rows, fastest id %d: %s\n", metrics.size(), metrics.empty() ? -1 : metrics[0].id,
                            ok ? "ok" : "FAILED");
                failed += !ok;
                // what Measure learnt survives in a file: a second object loads it and makes the same choice
                const std::string path = "/tmp/w4a16_dropin_tuning.txt";
                const int         saved = gemm.SaveTuning(path);
                GemmS4F16         other;
                const int         loaded = other.LoadTuning(path);
                std::printf("tuning file: saved %d, loaded %d: %s\n", saved, loaded, saved == 1 && loaded == 1 ? "ok" : "FAILED");
                failed += !(saved == 1 && loaded == 1);
            }
            (void)hipFree(X);
            (void)hipFree(R);
            (void)hipFree(C);
        }
        // the reference's error behaviour (gemm_s4_f16.cu:119,233)
        try {
            GemmS4F16 gemm;
            gemm.Run((half*)A, A, (const half*)A, Q, N, 4, K, 256, GemmS4F16::kGemm, -1, stream);
            std::printf("group size 256 was accepted: FAILED\n");
            ++failed;
        }
        catch (const std::runtime_error& e) {
            const bool ok = std::strcmp(e.what(), "unsupported group size") == 0;
            std::printf("group size 256: \"%s\" %s\n", e.what(), ok ? "ok" : "FAILED");
            failed += !ok;
        }
        std::printf(failed ? "drop-in checks FAILED: %d\n" : "drop-in checks passed\n", failed);
        return failed != 0;
    }
    catch (const std::exception& e) {
        std::printf("no GPU work done: %s\n", e.what());
        return 0;
    }
}
