// C++ face of the library-level boundary: the one CpuBackend method on the Q4_K path, with the
// reference's argument meaning, over the C ABI.  Header-only; link libmi355q4k_ggml.so.
//
// Mirrors CpuBackend::GgmlQuantizedMatrixView and CpuBackend::MatMulGgmlQuantizedTransB
// (core/include/densecore/backend/cpu_backend.h:91-99,293-300) and the Tensor fields they read
// (core/include/densecore/hal/tensor.h:280-289): shape[0] outermost, stride in ELEMENTS.
#pragma once
#include <array>
#include <cstddef>
#include <cstdint>

#include "mi355_q4k_ggml.h"

namespace densecore_amd {

enum class DType : int { F32 = 0, Other = 1 };

struct Tensor {
    void* data = nullptr;
    std::array<int64_t, 4> shape{0, 0, 0, 0};
    std::array<int64_t, 4> stride{0, 0, 0, 0};
    int ndim = 0;
    DType dtype = DType::F32;

    bool IsValid() const { return data != nullptr && ndim >= 1 && ndim <= 4; }
    static Tensor Matrix(float* data, int64_t rows, int64_t cols) {
        Tensor t;
        t.data = data;
        t.shape = {rows, cols, 0, 0};
        t.stride = {cols, 1, 0, 0};
        t.ndim = 2;
        return t;
    }
};

class Mi355Q4KBackend {
public:
    struct GgmlQuantizedMatrixView {
        const void* data = nullptr;
        int32_t type_id = -1;  // ggml_type; 12 (GGML_TYPE_Q4_K), 13 (GGML_TYPE_Q5_K) and 14 (GGML_TYPE_Q6_K) are accepted
        int64_t rows = 0;      // N
        int64_t cols = 0;      // K
        size_t row_bytes = 0;
        bool IsValid() const { return data != nullptr && type_id >= 0 && rows > 0 && cols > 0 && row_bytes > 0; }
    };

    // C[M,N] = A[M,K] . W[N,K]^T; false = rejected, C untouched
    // (core/src/backend/cpu_backend_quantized_matmul.cpp:150-175).
    bool MatMulGgmlQuantizedTransB(const Tensor& A, const GgmlQuantizedMatrixView& W, Tensor* C,
                                   int /*numa_node_id*/ = 0) const {
        if (!A.IsValid() || !W.IsValid() || !C || !C->IsValid() || A.dtype != DType::F32 || C->dtype != DType::F32 ||
            A.ndim != 2 || C->ndim != 2 || A.shape[1] != W.cols || C->shape[0] != A.shape[0] || C->shape[1] != W.rows ||
            A.stride[1] != 1 || C->stride[1] != 1)
            return false;
        return mq_matmul_ggml_quantized_transb(static_cast<const float*>(A.data), A.shape[0], A.shape[1], A.stride[0],
                                               W.data, W.type_id, W.rows, W.cols, W.row_bytes,
                                               static_cast<float*>(C->data), C->stride[0]) == 1;
    }
};

}  // namespace densecore_amd
