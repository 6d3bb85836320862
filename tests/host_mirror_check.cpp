// Drives frink_amd/host/frink_hip.hpp the way the reference's own seam tests drive a backend
// (crates/frink-core/src/weight_matrix/gpu_backend.rs:1093-1104, 1265).  Without arguments it
// needs no GPU; with --gpu it also launches a matvec and a batched GEMM and checks them against
// closed forms.  Prints one line per check; exit status 0 = all passed.
#include <cmath>
#include <cstdio>
#include <cstring>

#include "../frink_amd/host/frink_hip.hpp"

using namespace frink_hip;

static int failures = 0;
#define CHECK(cond, what)                                        \
    do {                                                         \
        bool ok_ = (cond);                                       \
        std::printf("%s  %s\n", ok_ ? "ok  " : "FAIL", what);    \
        if (!ok_) failures++;                                    \
    } while (0)

static uint16_t f16_pow2_bits(int e) {  // f16 bits of 2^e, -14 <= e <= 15
    return (uint16_t)((15 + e) << 10);
}

int main(int argc, char **argv) {
    const bool gpu = argc > 1 && std::strcmp(argv[1], "--gpu") == 0;

    // every kind a backend claims can actually be launched, and only those
    bool agree = true;
    int claimed = 0;
    for (QuantKind k : ALL_KINDS) {
        agree = agree && (Hip::matvec_kernel(k).has_value() == Hip::has_launch(k));
        if (Hip::matvec_kernel(k)) {
            claimed++;
            agree = agree && std::strcmp(*Hip::matvec_kernel(k), name(k)) == 0;
        }
        if (Hip::gemm_supported(k)) agree = agree && Hip::has_launch(k);
    }
    CHECK(agree, "matvec_kernel(kind) agrees with has_launch(kind) over all 23 kinds and names the kind");
    CHECK(claimed == 8 && Hip::has_launch(QuantKind::Q8_0) && Hip::has_launch(QuantKind::Q4K) &&
              Hip::has_launch(QuantKind::Q5K) && Hip::has_launch(QuantKind::Q6K) && Hip::has_launch(QuantKind::Q4_0) &&
              Hip::has_launch(QuantKind::Q5_0) && Hip::has_launch(QuantKind::IQ4XS) && Hip::has_launch(QuantKind::Mxfp4Gguf),
          "the eight kinds of this path have kernels");

    // None vs Some(Err)
    std::vector<uint8_t> w(34 * 4, 0);
    std::vector<float> x(32, 1.0f);
    CHECK(!Hip::launch_matvec(QuantKind::Q5_1, w.data(), w.size(), x.data(), x.size(), 4, 34).has_value(),
          "a kind without a kernel is None, not an error");
    auto bad = Hip::launch_matvec(QuantKind::Q8_0, w.data(), w.size(), x.data(), x.size(), 4, 35);
    CHECK(bad.has_value() && bad->is_err() && bad->error().status == FRK_ERR_SHAPE && !bad->error().message.empty(),
          "row_bytes that is not whole blocks is Some(Err) with a message");
    bad = Hip::launch_matvec(QuantKind::Q8_0, w.data(), w.size(), x.data(), 31, 4, 34);
    CHECK(bad.has_value() && bad->is_err() && bad->error().status == FRK_ERR_SHAPE, "a short activation is Some(Err)");
    bad = Hip::launch_matvec(QuantKind::Q8_0, w.data(), w.size(), x.data(), x.size(), 0, 34);
    CHECK(bad.has_value() && bad->is_err(), "rows == 0 is Some(Err)");
    auto mm = launch_mul_mm(QuantKind::Q4K, w.data(), w.size(), x.data(), x.size(), 4, 32, 1, 34);
    CHECK(mm.is_err(), "launch_mul_mm validates the shape before launching");
    auto wm = WeightMatrix::quantized(QuantKind::Q4K, w.data(), w.size(), 4, 32);
    CHECK(wm.is_err() && wm.error().status == FRK_ERR_SHAPE, "WeightMatrix::quantized rejects cols that are not whole blocks");
    CHECK(worth_a_gemm(2) && !worth_a_gemm(1), "worth_a_gemm: every batch >= 2");

    if (!gpu) {
        // forced off by the environment (set by the caller): no device is opened
        const char *env = std::getenv("FRINK_HIP");
        if (env && std::strcmp(env, "off") == 0) CHECK(!Hip::dense_enabled(), "FRINK_HIP=off disables the backend");
        std::printf("%d failure(s)\n", failures);
        return failures ? 1 : 0;
    }

    auto info = probe();
    CHECK(info.has_value() && info->gcn_arch.rfind("gfx950", 0) == 0, "probe finds a gfx950 device");
    CHECK(Hip::dense_enabled(), "dense_enabled after a successful probe");

    // Q8_0, 8 rows x 64 cols: row r has d = 2^-r and quants q[i] = (i % 7) - 3; x[i] = i % 5.
    // y[r] = 2^-r * sum_i q[i]*x[i], exact in f32.
    const size_t rows = 8, cols = 64, nb = cols / 32;
    std::vector<uint8_t> w8(rows * nb * 34);
    std::vector<float> xv(cols);
    long isum = 0;
    for (size_t i = 0; i < cols; i++) {
        xv[i] = (float)(i % 5);
        isum += ((long)(i % 7) - 3) * (long)(i % 5);
    }
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < nb; b++) {
            uint8_t *blk = &w8[(r * nb + b) * 34];
            uint16_t d = f16_pow2_bits(-(int)r);
            std::memcpy(blk, &d, 2);
            for (int i = 0; i < 32; i++) blk[2 + i] = (uint8_t)(int8_t)((int)((b * 32 + i) % 7) - 3);
        }
    auto y = Hip::launch_matvec(QuantKind::Q8_0, w8.data(), w8.size(), xv.data(), xv.size(), rows, nb * 34);
    bool exact = y.has_value() && y->is_ok();
    if (exact)
        for (size_t r = 0; r < rows; r++) exact = exact && y->value()[r] == std::ldexp((float)isum, -(int)r);
    CHECK(exact, "launch_matvec(Q8_0) equals the closed form exactly");

    // The batched entry point is batch-major.  A Q8_0 batch is quantized to Q8_0 activation blocks
    // first: with one value of 127*(t+1) in every block of token t the block scale is t+1 and the
    // quants are the values themselves, so the closed form is exact here too.
    std::vector<float> base(xv);
    base[0] = base[32] = 127.0f;
    long bsum = 0;
    for (size_t i = 0; i < cols; i++) bsum += ((long)(i % 7) - 3) * (long)base[i];
    std::vector<float> xb(3 * cols);
    for (size_t t = 0; t < 3; t++)
        for (size_t i = 0; i < cols; i++) xb[t * cols + i] = base[i] * (float)(t + 1);
    auto yb = launch_mul_mm(QuantKind::Q8_0, w8.data(), w8.size(), xb.data(), xb.size(), rows, cols, 3, nb * 34);
    bool major = yb.is_ok();
    if (major)
        for (size_t t = 0; t < 3; t++)
            for (size_t r = 0; r < rows; r++)
                major = major && yb.value()[t * rows + r] == std::ldexp((float)(bsum * (long)(t + 1)), -(int)r);
    CHECK(major, "launch_mul_mm output is out[token*n_rows + row]");

    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
