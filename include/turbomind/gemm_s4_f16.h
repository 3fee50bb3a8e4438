// Header-only C++ front end of libw4a16.so with the interface of TurboMind's
// turbomind::GemmS4F16 (src/turbomind/kernels/gemm_s_f16/gemm_s4_f16.h:17-56 in lmdeploy), so
// that LlamaLinear<T>::forwardInt4 (src/turbomind/models/llama/LlamaLinear.h:62-81) compiles
// against it unchanged: same class name, same Run/Measure argument order, same exceptions.
// Differences: the stream type is hipStream_t; Type gains kFusedAdd (value 2; 0 and 1 are
// unchanged) with an overload of Run that takes the residual.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <array>
#include <iomanip>
#include <iostream>
#include <limits>
#include <ostream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../w4a16.h"

namespace turbomind {

// metric.h:13-54.  Fields that describe CUDA occupancy modelling have no meaning here and
// are omitted; the ones a caller sorts or prints by are kept under the same names.
struct Metric {
    int                id;
    bool               feasible;
    bool               prefer;
    std::array<int, 3> cta_shape;  // {features, tokens, K slices per workgroup}
    int                kind;       // 0 decode kernel (column blocks), 1 MFMA prefill kernel, 2 decode kernel (strips)
    float              grid_size;
    int                best;
    float              time;       // milliseconds for `count` launches
    int                count;
};

// metric.h:56-110: one line per kernel configuration, in the order given.  The columns are this
// library's (tile, kernel family, grid, time per launch), not the CUDA occupancy model's.
inline void DumpMetrics(std::ostream& os, const std::vector<Metric>& metrics)
{
    static const char* const kKind[] = {"decode", "mfma", "strip"};
    os << std::setw(4) << "id" << std::setw(7) << "valid" << std::setw(9) << "kind" << std::setw(10) << "features"
       << std::setw(8) << "tokens" << std::setw(9) << "k_parts" << std::setw(8) << "grid" << std::setw(12) << "time_us"
       << std::setw(6) << "best" << "\n";
    for (const Metric& m : metrics) {
        os << std::setw(4) << m.id << std::setw(7) << m.feasible << std::setw(9)
           << (m.kind >= 0 && m.kind <= 2 ? kKind[m.kind] : "?") << std::setw(10) << m.cta_shape[0] << std::setw(8)
           << m.cta_shape[1] << std::setw(9) << m.cta_shape[2] << std::setw(8) << (int)m.grid_size << std::setw(12)
           << m.time * 1000 / m.count << std::setw(6) << (m.best ? "*" : "") << "\n";
    }
}

// gemm_s4_f16.h:15: when set, the next Measure prints its table to stderr once and clears the flag
// (gemm_s4_f16.cu:160-163)
inline bool g_dump_kernel_info_once = false;

class GemmS4F16 {
public:
    enum Type
    {
        kGemm,
        kFusedSiluFfn,
        kFusedAdd
    };

    GemmS4F16()
    {
        if (w4a16_create(&h_) != W4A16_OK) {
            throw std::runtime_error(w4a16_last_error());
        }
    }

    ~GemmS4F16()
    {
        w4a16_destroy(h_);
    }

    GemmS4F16(const GemmS4F16&) = delete;
    GemmS4F16& operator=(const GemmS4F16&) = delete;

    // gemm_s4_f16.h:41-51.  m = output features, n = tokens, k = input features.
    void Run(half*               C,
             const unsigned int* A,
             const half*         B,
             const half2*        Q,
             int                 m,
             int                 n,
             int                 k,
             int                 group_size,
             Type                type,
             int                 algo_id,
             hipStream_t         st)
    {
        Run(C, A, B, Q, nullptr, m, n, k, group_size, type, algo_id, st);
    }

    // with a residual for kFusedAdd: C = residual + B * W   (residual may alias C)
    void Run(half*               C,
             const unsigned int* A,
             const half*         B,
             const half2*        Q,
             const half*         residual,
             int                 m,
             int                 n,
             int                 k,
             int                 group_size,
             Type                type,
             int                 algo_id,
             hipStream_t         st)
    {
        const int rc = w4a16_gemm(h_, C, A, B, Q, residual, m, n, k, group_size, (int)type, algo_id, (void*)st);
        raise(rc);
    }

    // gemm_s4_f16.h:29-39
    void Measure(half*                C,
                 const unsigned int*  A,
                 const half*          B,
                 const half2*         Q,
                 int                  m,
                 int                  n,
                 int                  k,
                 int                  group_size,
                 Type                 type,
                 std::vector<Metric>& metrics,
                 hipStream_t          st,
                 const half*          residual = nullptr)
    {
        std::vector<w4a16_metric> raw(w4a16_algo_count());
        const int rc = w4a16_measure(h_, C, A, B, Q, residual, m, n, k, group_size, (int)type, raw.data(),
                                     (int)raw.size(), (void*)st);
        raise(rc);
        metrics.clear();
        for (int i = 0; i < rc; ++i) {
            const w4a16_metric& r = raw[i];
            Metric              x{};
            x.id        = r.id;
            x.feasible  = r.feasible != 0;
            x.prefer    = r.best != 0;
            x.cta_shape = {r.tile_n, r.tile_t, r.slices};
            x.kind      = r.kind;
            x.grid_size = (float)r.grid;
            x.best      = r.best;
            x.time      = r.ms;
            x.count     = r.count;
            metrics.push_back(x);
        }
        if (g_dump_kernel_info_once) {
            DumpMetrics(std::cerr, metrics);
            g_dump_kernel_info_once = false;
        }
    }

    // Extensions (the reference's Measure only reports): what Measure found fastest on this object, kept in a
    // text file across processes.  Both return the number of shapes written / taken over; LoadTuning throws
    // std::runtime_error for a file measured with another library version or on another GPU model.
    int SaveTuning(const std::string& path) const
    {
        const int rc = w4a16_save_tuning(h_, path.c_str());
        raise(rc);
        return rc;
    }

    int LoadTuning(const std::string& path)
    {
        const int rc = w4a16_load_tuning(h_, path.c_str());
        raise(rc);
        return rc;
    }

private:
    // gemm_s4_f16.cu:119,227,229,233: the same exception types and messages
    static void raise(int rc)
    {
        if (rc >= 0) return;
        switch (rc) {
            case W4A16_EGROUP: throw std::runtime_error("unsupported group size");
            case W4A16_ESHAPE: throw std::runtime_error("no feasible kernel found");
            case W4A16_EALGO: throw std::out_of_range(w4a16_last_error());
            default: throw std::runtime_error(w4a16_last_error());
        }
    }

    w4a16_handle* h_{};
};

}  // namespace turbomind
