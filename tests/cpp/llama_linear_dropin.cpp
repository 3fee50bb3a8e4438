// Compile-and-link check of the drop-in boundary: a LlamaLinear-shaped caller written against
// the reference's interface (src/turbomind/models/llama/LlamaLinear.h:15-87 in lmdeploy) using
// only the names the reference uses.  When run on a GPU box it also executes one GEMM through
// the class and prints the status; on a machine without a GPU the constructor throws and the
// program reports that instead.
#include "turbomind/format.h"
#include "turbomind/gemm_s4_f16.h"

#include <cstdio>
#include <type_traits>
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

int main()
{
    using namespace turbomind;
    static_assert(GemmS4F16::kGemm == 0 && GemmS4F16::kFusedSiluFfn == 1 && GemmS4F16::kFusedAdd == 2, "enum values");
    try {
        LlamaLinear<half> linear(nullptr);
        const int         K = 256, N = 64, T = 4, G = K / 128;
        uint32_t *        qw, *qz, *A;
        half *            s, *X, *C, *ws;
        half2*            Q;
        if (hipMalloc(&qw, K * N / 2) != hipSuccess) throw std::runtime_error("hipMalloc");
        (void)hipMalloc(&A, K * N / 2);
        (void)hipMalloc(&qz, G * N / 2);
        (void)hipMalloc(&s, G * N * 2);
        (void)hipMalloc(&ws, G * N * 2);
        (void)hipMalloc(&Q, G * N * 4);
        (void)hipMalloc(&X, T * K * 2);
        (void)hipMalloc(&C, T * N * 2);
        (void)hipMemset(qw, 0x33, K * N / 2);
        (void)hipMemset(qz, 0x33, G * N / 2);   // q == z  =>  output must be all zero
        (void)hipMemset(s, 0x3c, G * N * 2);
        (void)hipMemset(X, 0x3c, T * K * 2);
        convert_s4_k_m8(A, Q, ws, qw, s, qz, N, K, 128, nullptr);
        LlamaDenseWeight<half> w{(size_t)K, (size_t)N, A, WeightType::kINT4, nullptr, (half*)Q, 128};
        linear.forward(C, X, T, w);
        std::vector<unsigned short> out(T * N);
        (void)hipMemcpy(out.data(), C, T * N * 2, hipMemcpyDeviceToHost);
        int bad = 0;
        for (auto v : out) bad += (v & 0x7fff) != 0;
        std::printf("drop-in GEMM ran, non-zero outputs: %d\n", bad);
        return bad != 0;
    }
    catch (const std::exception& e) {
        std::printf("no GPU work done: %s\n", e.what());
        return 0;
    }
}
