// GPU parity through the C++ host mirror (include/gllm_hip_quant.hpp): host-slice calls with
// the reference's names and argument order, checked against the C oracle.
// Exit code 0 = all checks passed.  Needs a gfx950 device.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "gllm_hip_quant.hpp"
#include "gllmq_oracle.h"

namespace {

uint64_t rng_state = 0x9E3779B97F4A7C15ull;
uint64_t next_u64()
{
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
double uniform() { return (next_u64() >> 11) * (1.0 / 9007199254740992.0); }
float normal()
{
    const double u1 = uniform() + 1e-300, u2 = uniform();
    return static_cast<float>(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
}

// f32 -> f16 bits for positive normal values (enough for scales in (0.001, 0.05))
uint16_t f16_bits(float v)
{
    uint32_t b;
    std::memcpy(&b, &v, 4);
    const uint32_t e = ((b >> 23) & 0xFF) - 127 + 15, man = (b >> 13) & 0x3FF;
    return static_cast<uint16_t>((e << 10) | man);
}

// random blocks: every byte pattern is a valid block; the f16 scales get sane magnitudes
std::vector<uint8_t> random_weight(uint32_t dtype, size_t n, size_t k)
{
    const size_t bb = gq_block_bytes(dtype), rb = gq_row_bytes(dtype, k);
    std::vector<uint8_t> w(n * rb);
    for (auto &b : w) b = static_cast<uint8_t>(next_u64());
    for (size_t off = 0; off < w.size(); off += bb) {
        const uint16_t d = f16_bits(0.001f + 0.049f * static_cast<float>(uniform()));
        const uint16_t dm = f16_bits(0.001f + 0.049f * static_cast<float>(uniform()));
        if (dtype == 14) std::memcpy(&w[off + 208], &d, 2);
        else {
            std::memcpy(&w[off], &d, 2);
            if (dtype == 12 || dtype == 13) std::memcpy(&w[off + 2], &dm, 2);
        }
    }
    return w;
}

int failures = 0;
#define CHECK(cond, ...)                                                                      \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__);                                  \
            std::printf(__VA_ARGS__);                                                         \
            std::printf("\n");                                                                \
            ++failures;                                                                       \
        }                                                                                     \
    } while (0)

} // namespace

int main()
{
    using gllm::BackendError;
    using gllm::QuantType;
    gllm::HipBackend backend(0);
    if (backend.init_error()) {
        std::printf("init failed: %s\n", backend.init_error().message.c_str());
        return 2;
    }
    const QuantType kinds[] = { QuantType::Q8_0, QuantType::Q4K, QuantType::Q5K, QuantType::Q6K };
    for (QuantType qt : kinds) {
        const uint32_t dtype = static_cast<uint32_t>(qt);
        const size_t m = 3, n = 37, k = 1024;
        std::printf("quant type %u: dequantize + quantized_matmul %zux%zux%zu\n", dtype, m, n, k);
        std::fflush(stdout);
        CHECK(gllm::block_size(qt) == gq_block_size(dtype) && gllm::block_bytes(qt) == gq_block_bytes(dtype),
              "format constants differ for %u", dtype);
        const std::vector<uint8_t> w = random_weight(dtype, n, k);
        std::vector<float> x(m * k);
        for (auto &v : x) v = normal();

        // dequantize: bit-exact
        std::vector<float> deq(n * k, -1.0f), deq_ref(n * k, -2.0f);
        BackendError e = backend.dequantize(w.data(), w.size(), deq.data(), deq.size(), qt);
        CHECK(e.ok(), "dequantize: %s", e.message.c_str());
        gq_dequantize(w.data(), w.size(), deq_ref.data(), deq_ref.size(), dtype);
        CHECK(std::memcmp(deq.data(), deq_ref.data(), deq.size() * 4) == 0, "dequantize differs from the oracle");

        // quantized_matmul: rel-L2 <= 1e-4, |err| <= 1e-3 max|y| against f64 accumulation
        std::vector<float> y(m * n, NAN), y_ref(m * n);
        e = backend.quantized_matmul(w.data(), w.size(), x.data(), x.size(), y.data(), y.size(), qt, m, n, k);
        CHECK(e.ok(), "quantized_matmul: %s", e.message.c_str());
        gq_quantized_matmul(w.data(), x.data(), y_ref.data(), dtype, m, n, k, GQ_ACC_F64, 1);
        double num = 0, den = 0, worst = 0, ymax = 0;
        for (size_t i = 0; i < y.size(); ++i) {
            const double d = static_cast<double>(y[i]) - y_ref[i];
            num += d * d;
            den += static_cast<double>(y_ref[i]) * y_ref[i];
            worst = std::fmax(worst, std::fabs(d));
            ymax = std::fmax(ymax, std::fabs(static_cast<double>(y_ref[i])));
        }
        const double rel = std::sqrt(num / den);
        CHECK(rel <= 1e-4 && worst <= 1e-3 * ymax, "matmul rel_l2=%.3e worst=%.3e max|y|=%.3e", rel, worst, ymax);
        std::printf("  rel_l2 = %.3e\n", rel);

        // short output slice: an error of kind Other, nothing written
        e = backend.quantized_matmul(w.data(), w.size(), x.data(), x.size(), y.data(), m * n - 1, qt, m, n, k);
        CHECK(e.kind == BackendError::Kind::Other, "short output slice must be rejected");

        // quant_gather: the n rows as an embedding table, bit-exact, with and without a scale
        const uint32_t ids[5] = { 36, 0, 7, 7, 20 };
        const float scale = 32.0f; // sqrt(k)
        std::vector<float> rows(5 * k, -1.0f), rows_ref(5 * k, -2.0f);
        e = backend.quant_gather(w.data(), w.size(), qt, n, k, ids, 5, nullptr, rows.data(), rows.size());
        CHECK(e.ok(), "quant_gather: %s", e.message.c_str());
        gq_quant_gather(w.data(), dtype, n, k, ids, 5, 1.0f, 0, rows_ref.data());
        CHECK(std::memcmp(rows.data(), rows_ref.data(), rows.size() * 4) == 0, "quant_gather differs from the oracle");
        e = backend.quant_gather(w.data(), w.size(), qt, n, k, ids, 5, &scale, rows.data(), rows.size());
        CHECK(e.ok(), "scaled quant_gather: %s", e.message.c_str());
        gq_quant_gather(w.data(), dtype, n, k, ids, 5, scale, 1, rows_ref.data());
        CHECK(std::memcmp(rows.data(), rows_ref.data(), rows.size() * 4) == 0, "scaled quant_gather differs from the oracle");
        const uint32_t bad[1] = { 37 };
        e = backend.quant_gather(w.data(), w.size(), qt, n, k, bad, 1, nullptr, rows.data(), rows.size());
        CHECK(e.kind == BackendError::Kind::Other, "an id outside the table must be rejected");
    }
    // formats outside the four are Unimplemented, never a fallback (cpu_backend.rs:1020-1046)
    {
        std::vector<uint8_t> w(18 * 8);
        std::vector<float> x(256), y(1);
        BackendError e = backend.quantized_matmul(w.data(), w.size(), x.data(), x.size(), y.data(), y.size(),
                                                  QuantType::Q4_0, 1, 1, 256);
        CHECK(e.kind == BackendError::Kind::Unimplemented, "Q4_0 must be Unimplemented, got kind %d", static_cast<int>(e.kind));
        e = backend.dequantize(w.data(), w.size(), x.data(), x.size(), QuantType::Q2K);
        CHECK(e.kind == BackendError::Kind::Unimplemented, "Q2K dequantize must be Unimplemented");
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
