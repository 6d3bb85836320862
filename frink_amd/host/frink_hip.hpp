// C++ host side of the HIP backend: the shapes Frink's Rust seam has, over the C ABI.
//
// The reference's backend seam is a pair of traits with receiver-less members plus a few free
// launch functions (crates/frink-core/src/weight_matrix/gpu_backend.rs:90-195,
// crates/frink-cuda/src/gpu.rs:319-446, crates/frink-cuda/src/mul_mm_launch.rs:40-68).  This
// header gives the same names, argument meaning and error behaviour in C++17:
//
//   QuantKind, name()                 weight_matrix.rs:118-175, 264-290
//   BackendError                      gpu_backend.rs:90
//   Hip::{NAME, GEMM_FALLBACK, MATVEC_FALLBACK, matvec_kernel, gemm_supported,
//         dense_enabled, has_launch, launch_matvec}       BackendCaps + BackendDispatch
//   launch_mul_mm, worth_a_gemm       mul_mm_launch.rs:40-68, mul_mm.rs:634-638
//   probe                             gpu.rs:79-145
//   WeightMatrix (Quantized)          weight_matrix.rs:780-787: apply / apply_batch on resident weights
//   route_top_k_softmax, MoeExperts   frink-moe/src/lib.rs:567-589, decoder/ffn_batch.rs:343-434
//
// Option<Result<..>> becomes std::optional<Result<..>>: nullopt = "no kernel for this kind",
// an error value = "the kernel exists and the launch failed".  Nothing here throws.
#pragma once

#include <cstdint>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "../../include/frink_hip.h"

namespace frink_hip {

// ggml type ids; PTQ1_0 is Frink's own kind and has none.
enum class QuantKind : int {
    Q8_0 = 8, Q4_0 = 2, Q4K = 12, Q5K = 13, Q6K = 14, Q2K = 10, Q3K = 11, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7,
    Q8_1 = 9, IQ4NL = 20, IQ4XS = 23, IQ1S = 19, IQ2XXS = 16, IQ3XXS = 18, IQ2XS = 17, IQ2S = 22,
    IQ3S = 21, IQ1M = 29, Mxfp4Gguf = 39, Tq1_0 = 34, Ptq1_0 = -1,
};

inline constexpr QuantKind ALL_KINDS[23] = {
    QuantKind::Q8_0, QuantKind::Q4_0, QuantKind::Q4K, QuantKind::Q5K, QuantKind::Q6K, QuantKind::Q2K,
    QuantKind::Q3K, QuantKind::Q4_1, QuantKind::Q5_0, QuantKind::Q5_1, QuantKind::Q8_1, QuantKind::IQ4NL,
    QuantKind::IQ4XS, QuantKind::IQ1S, QuantKind::IQ2XXS, QuantKind::IQ3XXS, QuantKind::IQ2XS,
    QuantKind::IQ2S, QuantKind::IQ3S, QuantKind::IQ1M, QuantKind::Mxfp4Gguf, QuantKind::Tq1_0,
    QuantKind::Ptq1_0,
};

inline const char *name(QuantKind k) {
    switch (k) {
    case QuantKind::Q8_0: return "Q8_0";
    case QuantKind::Q4_0: return "Q4_0";
    case QuantKind::Q4K: return "Q4_K";
    case QuantKind::Q5K: return "Q5_K";
    case QuantKind::Q6K: return "Q6_K";
    case QuantKind::Q2K: return "Q2_K";
    case QuantKind::Q3K: return "Q3_K";
    case QuantKind::Q4_1: return "Q4_1";
    case QuantKind::Q5_0: return "Q5_0";
    case QuantKind::Q5_1: return "Q5_1";
    case QuantKind::Q8_1: return "Q8_1";
    case QuantKind::IQ4NL: return "IQ4_NL";
    case QuantKind::IQ4XS: return "IQ4_XS";
    case QuantKind::IQ1S: return "IQ1_S";
    case QuantKind::IQ2XXS: return "IQ2_XXS";
    case QuantKind::IQ3XXS: return "IQ3_XXS";
    case QuantKind::IQ2XS: return "IQ2_XS";
    case QuantKind::IQ2S: return "IQ2_S";
    case QuantKind::IQ3S: return "IQ3_S";
    case QuantKind::IQ1M: return "IQ1_M";
    case QuantKind::Mxfp4Gguf: return "MXFP4";
    case QuantKind::Tq1_0: return "TQ1_0";
    case QuantKind::Ptq1_0: return "PTQ1_0";
    }
    return "?";
}

// The one shape the seam carries: a message callers print before falling back.
struct BackendError {
    std::string message;
    int status = 0;  // the C ABI's status code, for tests
};

template <class T>
class Result {
  public:
    Result(T v) : ok_(true), value_(std::move(v)) {}
    Result(BackendError e) : ok_(false), error_(std::move(e)) {}
    bool is_ok() const { return ok_; }
    bool is_err() const { return !ok_; }
    const T &value() const { return value_; }
    T &value() { return value_; }
    const BackendError &error() const { return error_; }

  private:
    bool ok_;
    T value_{};
    BackendError error_{};
};

inline BackendError last_error(int status) { return BackendError{frk_hip_last_error(), status}; }

struct HipInfo {  // frink_cuda::gpu::CudaInfo
    int device_count;
    std::string first_device_name, gcn_arch;
    int compute_units;
    uint64_t total_vram_bytes, free_vram_bytes;
};

// Never aborts on a GPU-less host: nullopt there.
inline std::optional<HipInfo> probe() {
    frk_device_info i;
    if (frk_hip_probe(&i) != FRK_OK) return std::nullopt;
    return HipInfo{i.device_count, i.name, i.gcn_arch, i.compute_units, i.total_vram_bytes, i.free_vram_bytes};
}

// The backend's unit type: BackendCaps + BackendDispatch.
struct Hip {
    static constexpr const char *NAME = "HIP";
    static constexpr const char *GEMM_FALLBACK = "HIP N x matvec batch";
    static constexpr const char *MATVEC_FALLBACK = "CPU";

    static std::optional<const char *> matvec_kernel(QuantKind kind) {
        const char *n = frk_hip_matvec_kernel((int)kind);
        return n ? std::optional<const char *>(n) : std::nullopt;
    }
    static bool gemm_supported(QuantKind kind) { return frk_hip_gemm_supported((int)kind) != 0; }
    static bool dense_enabled() { return frk_hip_dense_enabled() != 0; }
    static bool has_launch(QuantKind kind) { return frk_hip_has_launch((int)kind) != 0; }

    static std::optional<Result<std::vector<float>>> launch_matvec(QuantKind kind, const uint8_t *weights,
                                                                   size_t weights_len, const float *x, size_t x_len,
                                                                   size_t rows, size_t row_bytes) {
        if (!has_launch(kind)) return std::nullopt;
        std::vector<float> out(rows);
        int rc = frk_hip_launch_matvec((int)kind, weights, weights_len, x, x_len, rows, row_bytes, out.data());
        if (rc != FRK_OK) return Result<std::vector<float>>(last_error(rc));
        return Result<std::vector<float>>(std::move(out));
    }
};

inline bool worth_a_gemm(size_t batch) { return frk_hip_worth_a_gemm(batch) != 0; }

// out[token*n_rows + row]
inline Result<std::vector<float>> launch_mul_mm(QuantKind kind, const uint8_t *weights, size_t weights_len,
                                                const float *x_batch, size_t x_len, size_t n_rows, size_t n_cols,
                                                size_t batch, size_t row_bytes) {
    std::vector<float> out(n_rows * batch);
    int rc = frk_hip_launch_mul_mm((int)kind, weights, weights_len, x_batch, x_len, n_rows, n_cols, batch, row_bytes,
                                   out.data());
    if (rc != FRK_OK) return last_error(rc);
    return out;
}

// WeightMatrix::Quantized{data, rows, cols, kind} whose bytes are resident in HBM.  `data` is
// borrowed for the constructor call only.  Move-only; releases the handle on destruction.
class WeightMatrix {
  public:
    static Result<WeightMatrix> quantized(QuantKind kind, const uint8_t *data, size_t len, size_t rows, size_t cols) {
        frk_weights *h = nullptr;
        int rc = frk_hip_weights_register((int)kind, data, len, rows, cols, &h);
        if (rc != FRK_OK) return last_error(rc);
        return WeightMatrix(h, kind, rows, cols);
    }
    WeightMatrix() = default;
    WeightMatrix(WeightMatrix &&o) noexcept { *this = std::move(o); }
    WeightMatrix &operator=(WeightMatrix &&o) noexcept {
        if (this != &o) {
            reset();
            h_ = o.h_, kind_ = o.kind_, rows_ = o.rows_, cols_ = o.cols_;
            o.h_ = nullptr;
        }
        return *this;
    }
    WeightMatrix(const WeightMatrix &) = delete;
    WeightMatrix &operator=(const WeightMatrix &) = delete;
    ~WeightMatrix() { reset(); }

    size_t rows() const { return rows_; }
    size_t cols() const { return cols_; }
    QuantKind kind() const { return kind_; }
    const frk_weights *handle() const { return h_; }

    // y[rows] = W x, operands in HBM, asynchronous on `stream` (WeightMatrix::apply_gpu)
    Result<bool> apply_dev(const float *x_dev, float *y_dev, void *stream) const {
        int rc = frk_hip_gemv_dev(h_, x_dev, y_dev, FRK_ACT_F32, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }
    // y[batch][rows] (WeightMatrix::apply_batch)
    Result<bool> apply_batch_dev(const float *x_dev, size_t batch, float *y_dev, void *stream) const {
        int rc = frk_hip_gemm_dev(h_, x_dev, batch, y_dev, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }

    // y[pairs][rows / n_groups]: this matrix as n_groups stacked groups, pair p of group g (group_off[g] <= p <
    // group_off[g + 1]) times row gather[p] of x (row p without a gather list); everything on the device
    // (enqueue_mul_mm_grouped_dev, crates/frink-cuda/src/mul_mm_launch.rs:391-470)
    Result<bool> apply_grouped_dev(size_t n_groups, const int32_t *group_off_dev, const int32_t *gather_dev, const float *x_dev,
                                   size_t x_rows, size_t pairs, float *y_dev, void *stream) const {
        int rc = frk_hip_gemm_grouped_dev(h_, n_groups, group_off_dev, gather_dev, x_dev, x_rows, pairs, y_dev, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }

    // Q5_0 / IQ4_XS / MXFP4: the rows decoded for the matrix cores kept beside the resident copy (no counterpart in
    // the reference, whose GEMM dequantizes inside the kernel: crates/frink-cuda/src/mul_mm.rs:146-205)
    Result<bool> keep_decoded(void *stream) {
        int rc = frk_hip_weights_keep_decoded(h_, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }

  private:
    WeightMatrix(frk_weights *h, QuantKind k, size_t r, size_t c) : h_(h), kind_(k), rows_(r), cols_(c) {}
    void reset() {
        if (h_) frk_hip_weights_release(h_);
        h_ = nullptr;
    }
    frk_weights *h_ = nullptr;
    QuantKind kind_ = QuantKind::Q8_0;
    size_t rows_ = 0, cols_ = 0;
};

// BatchActs::Q8K (crates/frink-core/src/weight_matrix.rs:757-768): a batch's activations quantized once for any number
// of matrices of `cols` columns (quantize_batch_acts, :2348-2426), at any batch size up to max_batch.  Move-only.
class BatchActs {
  public:
    static Result<BatchActs> with_room_for(size_t max_batch, size_t cols) {
        frk_batch_acts *h = nullptr;
        int rc = frk_hip_batch_acts_create(max_batch, cols, &h);
        if (rc != FRK_OK) return last_error(rc);
        return BatchActs(h);
    }
    BatchActs() = default;
    BatchActs(BatchActs &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    BatchActs &operator=(BatchActs &&o) noexcept {
        if (this != &o) {
            if (h_) frk_hip_batch_acts_release(h_);
            h_ = o.h_;
            o.h_ = nullptr;
        }
        return *this;
    }
    BatchActs(const BatchActs &) = delete;
    BatchActs &operator=(const BatchActs &) = delete;
    ~BatchActs() {
        if (h_) frk_hip_batch_acts_release(h_);
    }
    Result<bool> quantize_dev(const float *x_dev, size_t batch, void *stream) {
        int rc = frk_hip_quantize_batch_acts_dev(h_, x_dev, batch, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }
    // WeightMatrix::apply_batch_with_acts (:2481-2487): y[batch][rows], bit for bit apply_batch_dev's result
    Result<bool> apply_dev(const WeightMatrix &w, float *y_dev, void *stream) const {
        int rc = frk_hip_gemm_acts_dev(w.handle(), h_, y_dev, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }

  private:
    explicit BatchActs(frk_batch_acts *h) : h_(h) {}
    frk_batch_acts *h_ = nullptr;
};

// One MoE layer's experts, stacked per projection (ExpertWeights{gate, up, down} x n_experts).
struct MoeExperts {
    WeightMatrix gate, up, down;
    size_t n_experts = 0;

    // Decoder::moe_ffn_batch: ids/weights are one RoutingDecision per token, [batch][k]
    Result<bool> ffn_batch_dev(const float *x_dev, size_t batch, const int32_t *ids_dev, const float *weights_dev,
                               size_t k, float *out_dev, void *stream) const {
        int rc = frk_hip_moe_ffn_dev(gate.handle(), up.handle(), down.handle(), n_experts, x_dev, batch, ids_dev,
                                     weights_dev, k, out_dev, stream);
        if (rc != FRK_OK) return last_error(rc);
        return true;
    }
};

}  // namespace frink_hip
