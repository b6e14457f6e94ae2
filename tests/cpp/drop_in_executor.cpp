// A program written against the ark:: C++ API only (<ark/ark.hpp>, linked with
// -larkmi): what a user of the reference's headers would compile unchanged.
// It follows how the reference's op tests drive an executor
// (ark/ops/ops_test_common.cpp:34-224, ark/api/executor_test.cpp): build a Model,
// run it through DefaultExecutor, compare with a host loop.
//
// Operand values are multiples of 1/2 in [-1, 1] and K = 128, so every product sum is
// a multiple of 1/4 below 2^9 and exact in fp16: the comparison is bit for bit.
#include <ark/ark.hpp>
// the single headers a program may name instead of the umbrella one
#include <ark/init.hpp>
#include <ark/log.hpp>
#include <ark/model_ref.hpp>
#include <ark/random.hpp>
#include <ark/version.hpp>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

static uint16_t half_bits(float v) {
    // exact for the values used here (|v| <= 512, multiples of 1/4)
    if (v == 0.f) return 0;
    uint32_t u;
    std::memcpy(&u, &v, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int32_t exp = (int32_t)((u >> 23) & 0xff) - 127 + 15;
    return (uint16_t)(sign | ((uint32_t)exp << 10) | ((u >> 13) & 0x3ffu));
}

static int fails = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
            ++fails;                                                        \
        }                                                                   \
    } while (0)

int main() {
    ark::init();
    static_assert(ARK_VERSION == ARK_MAJOR * 10000 + ARK_MINOR * 100 + ARK_PATCH, "version macros");
    EXPECT(!ark::version().empty());
    ark::log(ark::INFO, __FILE__, __LINE__, "drop_in_executor: start");  // goes to the log stream
    ark::log(ark::DEBUG, __FILE__, __LINE__, "below the default level: not printed");
    const int M = 256, N = 256, K = 128;
    std::vector<float> a((size_t)M * K), b((size_t)K * N);
    ark::srand(42);
    for (auto &v : a) v = (float)(ark::rand() % 5 - 2) * 0.5f;
    for (auto &v : b) v = (float)(ark::rand() % 5 - 2) * 0.5f;
    std::vector<uint16_t> ah(a.size()), bh(b.size());
    for (size_t i = 0; i < a.size(); ++i) ah[i] = half_bits(a[i]);
    for (size_t i = 0; i < b.size(); ++i) bh[i] = half_bits(b[i]);

    ark::Model m;
    ark::Tensor ta = m.tensor({M, K}, ark::FP16), tb = m.tensor({K, N}, ark::FP16);
    ark::Tensor tc = m.matmul(ta, tb);
    ark::Tensor td = m.add(tc, 1.0f);
    EXPECT(tc.shape() == ark::Dims(M, N));

    // the state machine of the reference: launch() before compile() is a usage error
    {
        ark::Planner planner(m, 0);
        ark::Executor bare(0, nullptr, "bare", planner.plan());
        bool thrown = false;
        try {
            bare.launch();
        } catch (const ark::InvalidUsageError &) {
            thrown = true;
        }
        EXPECT(thrown);
    }

    int rule_calls = 0;
    std::vector<ark::Planner::ConfigRule> rules = {
        [&rule_calls](const std::string &, const std::string &arch) -> std::string {
            ++rule_calls;
            if (arch != "ROCM_950") std::printf("unexpected architecture %s\n", arch.c_str());
            return "";  // decline: the defaults apply
        }};
    ark::DefaultExecutor exe(m, 0, nullptr, rules);
    EXPECT(rule_calls == 2);
    exe.compile();
    exe.tensor_write(ta, ah);
    exe.tensor_write(tb, bh);
    exe.launch();
    exe.run(3);
    exe.wait();
    std::vector<uint16_t> ch((size_t)M * N), dh((size_t)M * N);
    exe.tensor_read(tc, ch);
    exe.tensor_read(td, dh);
    const float ms = exe.stop();
    EXPECT(ms > 0.f);

    size_t bad = 0;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = 0.f;
            for (int k = 0; k < K; ++k) acc += a[(size_t)i * K + k] * b[(size_t)k * N + j];
            if (ch[(size_t)i * N + j] != half_bits(acc)) ++bad;
            if (dh[(size_t)i * N + j] != half_bits(acc + 1.0f)) ++bad;
        }
    EXPECT(bad == 0);

    // a byte count that does not match the tensor is refused (executor.cpp:799-804)
    bool thrown = false;
    try {
        std::vector<uint16_t> small(16);
        exe.tensor_read(tc, small);
    } catch (const ark::InvalidUsageError &) {
        thrown = true;
    }
    EXPECT(thrown);
    exe.destroy();
    EXPECT(exe.destroyed());

    if (fails) return 1;
    std::printf("drop_in_executor: OK (%d x %d x %d fp16 matmul + add, bit-exact, %.3f ms)\n", M, N, K, ms);
    return 0;
}
