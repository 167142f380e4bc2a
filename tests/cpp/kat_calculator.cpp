// Known-answer tests of the C++ surface (include/mme_hip_calculator.h) written the way the reference's own unit tests
// drive CPUCalculator (mme/tests/unit_tests/mme_unit_test.cpp:67-172, 394-519, 539-575): same shapes, values and expectations,
// host tensors, synchronous calls.  Needs a GPU.  Prints one line per case and exits non-zero on the first failure.
#include "mme_hip_calculator.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <vector>

using MmeHip::Calculator;
using MmeHip::MMEStackException;
using MmeHip::Tensor;
typedef Tensor::SizeArray SizeArray;

static int failures = 0;
#define EXPECT(cond)                                                                                                                       \
    do                                                                                                                                     \
    {                                                                                                                                      \
        if (!(cond))                                                                                                                       \
        {                                                                                                                                  \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                                                \
            failures++;                                                                                                                    \
        }                                                                                                                                  \
    } while (0)

static uint16_t bf16_of(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static float float_of_bf16(uint16_t h)
{
    const uint32_t u = (uint32_t) h << 16;
    float          f;
    std::memcpy(&f, &u, 4);
    return f;
}

// mme_unit_test.cpp:67-82
static void reference_gemm_simple_test_fp32(Calculator& calculator)
{
    std::vector<float> a(5, 10.0f), b(5, 10.0f), y(1, 0.0f);
    Tensor             ta({5, 1, 1, 1, 1}, 2, MME_HIP_FP32, a.data()), tb({1, 5, 1, 1, 1}, 2, MME_HIP_FP32, b.data()),
        ty({1, 1, 1, 1, 1}, 2, MME_HIP_FP32, y.data());
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
    EXPECT(y[0] == 500.0f);
}

// mme_unit_test.cpp:108-125
static void reference_gemm_simple_test_bf16(Calculator& calculator)
{
    std::vector<uint16_t> a(5, bf16_of(10.0f)), b(5, bf16_of(10.0f));
    std::vector<float>    y(1, 0.0f);
    Tensor ta({5, 1, 1, 1, 1}, 2, MME_HIP_BF16, a.data()), tb({1, 5, 1, 1, 1}, 2, MME_HIP_BF16, b.data()), ty({1, 1, 1, 1, 1}, 2, MME_HIP_FP32, y.data());
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
    EXPECT(y[0] == 500.0f);
}

// mme_unit_test.cpp:127-145.  The reference's test runs on Gaudi2 with e_type_fp32_ieee operands; Gaudi3 registers no
// worker for that type (mme_reference_impl.cpp:189-197), so here the operands are e_type_fp32 and the ieee type must throw.
static void reference_gemm_2d_test_fp32(Calculator& calculator)
{
    std::vector<float> a(25, 10.0f), b(25, 5.0f), y(25, 0.0f);
    Tensor ta({5, 5, 1, 1, 1}, 2, MME_HIP_FP32, a.data()), tb({5, 5, 1, 1, 1}, 2, MME_HIP_FP32, b.data()), ty({5, 5, 1, 1, 1}, 2, MME_HIP_FP32, y.data());
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
    for (int i = 0; i < 25; i++) EXPECT(y[i] == 250.0f);
    bool thrown = false;
    try
    {
        Tensor ia({5, 5, 1, 1, 1}, 2, MME_HIP_FP32_IEEE, a.data()), ib({5, 5, 1, 1, 1}, 2, MME_HIP_FP32_IEEE, b.data());
        calculator.doBatchGemm(ty, ia, ib, MME_HIP_OP_AB);
    }
    catch (const MMEStackException& e)
    {
        thrown = std::strstr(e.what(), "not registered") != nullptr;
    }
    EXPECT(thrown);
}

// mme_unit_test.cpp:147-172: GEMM, then doActivation to bf16
static void reference_gemm_2d_test_bf16(Calculator& calculator)
{
    std::vector<uint16_t> a(25, bf16_of(10.0f)), b(25, bf16_of(5.0f)), y(25, 0);
    std::vector<float>    acc(25, 0.0f);
    Tensor ta({5, 5, 1, 1, 1}, 2, MME_HIP_BF16, a.data()), tb({5, 5, 1, 1, 1}, 2, MME_HIP_BF16, b.data());
    Tensor tacc({5, 5, 1, 1, 1}, 2, MME_HIP_FP32, acc.data());
    calculator.doBatchGemm(tacc, ta, tb, MME_HIP_OP_AB);
    auto pY = std::make_shared<Tensor>(SizeArray {5, 5, 1, 1, 1}, 2, MME_HIP_BF16, y.data());
    auto pAcc = std::make_shared<Tensor>(tacc);
    calculator.doActivation(pY, pAcc, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false);
    for (int i = 0; i < 25; i++) EXPECT(float_of_bf16(y[i]) == 250.0f);
}

// mme_unit_test.cpp:394-408 and 467-481: the two conversions whose codes the reference's tests spell out
static void fp8_convert(Calculator& calculator)
{
    float   v143 = -0.25f, v152 = -0.5f;
    uint8_t c143 = 0, c152 = 0;
    auto    acc143 = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &v143);
    auto    out143 = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP8_143, &c143, 3u);
    calculator.doActivation(out143, acc143, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false);
    EXPECT(c143 == 0x88);
    auto acc152 = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &v152);
    auto out152 = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP8_152, &c152, 15u);
    calculator.doActivation(out152, acc152, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false);
    EXPECT(c152 == 0xB8);
}

// mme_unit_test.cpp:425-447 and 498-519: 0.25 * -0.5 summed twice, both fp8 flavours at their usual biases
static void reference_gemm_simple_test_fp8(Calculator& calculator)
{
    // fp8_143, bias 7: 0.25 = 2^(5-7) -> 0x28, -0.5 = -2^(6-7) -> 0xB0; fp8_152, bias 15: 0.25 = 2^(13-15) -> 0x34, -0.5 -> 0xB8
    const struct
    {
        int      type;
        unsigned bias;
        uint8_t  a, b;
    } flavours[] = {{MME_HIP_FP8_143, 7u, 0x28, 0xB0}, {MME_HIP_FP8_152, 15u, 0x34, 0xB8}};
    for (const auto& f : flavours)
    {
        std::vector<uint8_t> a(2, f.a), b(2, f.b);
        std::vector<float>   y(1, 0.0f);
        Tensor ta({2, 1, 1, 1, 1}, 2, f.type, a.data(), f.bias), tb({1, 2, 1, 1, 1}, 2, f.type, b.data(), f.bias), ty({1, 1, 1, 1, 1}, 2, MME_HIP_FP32, y.data());
        calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
        EXPECT(y[0] == 0.25f * -0.5f * 2);
    }
}

// fp16: the conversions the reference's unit test spells out (mme_unit_test.cpp:49-65: the largest fp16 is 0x7BFF =
// 65504 = fp32 0x477FE000, reached from the largest float with clipping; 0x7C00 is infinity) and the 10 * 10 dot product
// of its fp16 GEMM test (:544-575) over 128 terms
static void fp16_convert_and_gemm(Calculator& calculator)
{
    float    big = 3.402823466e38f, ten = 10.0f;
    uint16_t c_big = 0, c_inf = 0, c_ten = 0;
    auto     acc = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &big);
    auto     out = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP16, &c_big, 15u);
    calculator.doActivation(out, acc, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false, MME_HIP_RM_NEAREST_EVEN, nullptr, true);
    EXPECT(c_big == 0x7BFF);
    out = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP16, &c_inf, 15u);
    calculator.doActivation(out, acc, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false);
    EXPECT(c_inf == 0x7C00);
    acc = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &ten);
    out = std::make_shared<Tensor>(SizeArray {1, 1, 1, 1, 1}, 2, MME_HIP_FP16, &c_ten, 15u);
    calculator.doActivation(out, acc, std::shared_ptr<Tensor>(), std::shared_ptr<Tensor>(), false);
    EXPECT(c_ten == 0x4900);

    const unsigned        M = 2, N = 4, K = 128;
    std::vector<uint16_t> a(M * K, 0x4900), b(K * N, 0x4900), u(K * N, 0);
    std::vector<float>    y(M * N, 0.0f);
    Tensor ta({K, M, 1, 1, 1}, 2, MME_HIP_FP16, a.data(), 15u), tb({N, K, 1, 1, 1}, 2, MME_HIP_FP16, b.data(), 15u), ty({N, M, 1, 1, 1}, 2, MME_HIP_FP32, y.data());
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
    for (float v : y) EXPECT(v == 12800.0f);
    // the same value in unsigned fp16 (bias 31: 10 = 1.25 * 2^3 -> exponent 34, mantissa 0x100) mixes with fp16
    for (auto& v : u) v = (uint16_t) ((34u << 10) | 0x100u);
    Tensor tu({N, K, 1, 1, 1}, 2, MME_HIP_UFP16, u.data(), 31u);
    std::fill(y.begin(), y.end(), 0.0f);
    calculator.doBatchGemm(ty, ta, tu, MME_HIP_OP_AB);
    for (float v : y) EXPECT(v == 12800.0f);
}

// tf32 operands are rounded from fp32 on entry: the largest float becomes infinity unless clipFp is given
// (Gaudi3Tf32Fma, chip_fma/gaudi3_fma.cpp:237-272)
static void tf32_operand_clip(Calculator& calculator)
{
    float  a[2] = {3.402823466e38f, 0.0f}, b[2] = {7.52316385e-37f /* 2^-120 */, 1.0f}, y = 0.0f;
    Tensor ta({2, 1, 1, 1, 1}, 2, MME_HIP_TF32, a), tb({1, 2, 1, 1, 1}, 2, MME_HIP_TF32, b), ty({1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &y);
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB);
    EXPECT(std::isinf(y) && y > 0);
    calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB, MME_HIP_RM_NEAREST_EVEN, true);
    EXPECT(std::isfinite(y) && y > 255.0f && y < 256.0f); // 0x7F7FE000 * 2^-120 = (2 - 2^-10) * 2^7
}

// doMemoryWrite with a reduction, through shared pointers like the reference's callers (mme_reference.h:174-178): values
// chosen so that the result is known in closed form
static void memory_write_reductions(Calculator& calculator)
{
    // fp32 add, nearest even: 1 + 2^-24 is a tie and stays 1; round up makes it the next float; max_0 clamps a negative sum
    std::vector<float> mem = {1.0f, 1.0f, -3.0f, 2.5f}, out = {5.9604645e-08f, 5.9604645e-08f, 1.0f, -1.0f};
    auto               m = std::make_shared<Tensor>(SizeArray {4, 1, 1, 1, 1}, 1, MME_HIP_FP32, mem.data());
    auto               o = std::make_shared<Tensor>(SizeArray {4, 1, 1, 1, 1}, 1, MME_HIP_FP32, out.data());
    calculator.doMemoryWrite(m, o, MME_HIP_REDUCTION_ADD, MME_HIP_REDUCTION_RM_NEAREST_EVEN);
    EXPECT(mem[0] == 1.0f && mem[2] == -2.0f && mem[3] == 1.5f);
    mem = {1.0f, 1.0f, -3.0f, 2.5f};
    calculator.doMemoryWrite(m, o, MME_HIP_REDUCTION_ADD, MME_HIP_REDUCTION_RM_UP);
    EXPECT(mem[0] == std::nextafter(1.0f, 2.0f) && mem[2] == -2.0f);
    mem = {1.0f, 1.0f, -3.0f, 2.5f};
    calculator.doMemoryWrite(m, o, MME_HIP_REDUCTION_MAX_0, MME_HIP_REDUCTION_RM_NEAREST_EVEN);
    EXPECT(mem[2] == 0.0f && mem[3] == 1.5f);
    mem = {1.0f, 1.0f, -3.0f, 2.5f};
    calculator.doMemoryWrite(m, o, MME_HIP_REDUCTION_MIN);
    EXPECT(mem[0] == 5.9604645e-08f && mem[2] == -3.0f && mem[3] == -1.0f);
    // bf16 sub: 1 - 2^-9 needs a ninth significant bit: nearest even gives 1, toward zero the bf16 below 1
    std::vector<uint16_t> m16 = {bf16_of(1.0f), bf16_of(1.0f)}, o16 = {bf16_of(0.001953125f), bf16_of(0.001953125f)};
    auto                  mb = std::make_shared<Tensor>(SizeArray {2, 1, 1, 1, 1}, 1, MME_HIP_BF16, m16.data());
    auto                  ob = std::make_shared<Tensor>(SizeArray {2, 1, 1, 1, 1}, 1, MME_HIP_BF16, o16.data());
    calculator.doMemoryWrite(mb, ob, MME_HIP_REDUCTION_SUB, MME_HIP_REDUCTION_RM_NEAREST_EVEN);
    EXPECT(float_of_bf16(m16[0]) == 1.0f);
    m16 = {bf16_of(1.0f), bf16_of(1.0f)};
    calculator.doMemoryWrite(mb, ob, MME_HIP_REDUCTION_SUB, MME_HIP_REDUCTION_RM_TO_ZERO);
    EXPECT(float_of_bf16(m16[0]) == 0.99609375f);
    // reduction none copies
    calculator.doMemoryWrite(mb, ob);
    EXPECT(m16[0] == o16[0] && m16[1] == o16[1]);
}

// mme_unit_test.cpp:84-106: the Matrix form of the 5-term product, 1 x 5 times 5 x 1
static void reference_gemm_api_simple_test_fp32(Calculator& calculator)
{
    std::vector<float> data(5, 10.0f);
    MmeHip::Matrix     a(MME_HIP_FP32, 1, 5, data.data()), b(MME_HIP_FP32, 5, 1, data.data()), y(MME_HIP_FP32, 1, 1);
    calculator.doGemm(y, a, b, false, false);
    float got;
    std::memcpy(&got, y.data(), 4);
    EXPECT(got == 500.0f);
}

// mme_unit_test.cpp:539-575: fp16 operands, A handed in transposed (128 x 128), B 128 x 256, every element 10.  The
// reference's test asserts nothing; the values follow from the arithmetic: 128 products of 10 * 10 with the IEEE exponent
// bias, and with the call's default bias 0 every operand is 10 * 2^15.  All four transpose flags on a matrix with
// distinct entries: y = op(A) op(B) against a host loop.
static void reference_gemm_api(Calculator& calculator)
{
    const unsigned        M = 128, K = 128, N = 256;
    std::vector<uint16_t> da(K * M, 0x4900), db(K * N, 0x4900); // fp16 10.0
    MmeHip::Matrix        a(MME_HIP_FP16, K, M, da.data()), b(MME_HIP_FP16, K, N, db.data()), y(MME_HIP_FP32, M, N);
    calculator.doGemm(y, a, b, true, false, MME_HIP_RM_NEAREST_EVEN, 15, 15);
    const float* out = (const float*) y.data();
    bool         all = true;
    for (unsigned i = 0; i < M * N; i++) all = all && out[i] == 12800.0f;
    EXPECT(all);
    calculator.doGemm(y, a, b, true, false);
    all = true;
    for (unsigned i = 0; i < M * N; i++) all = all && out[i] == 12800.0f * 1073741824.0f;
    EXPECT(all);
    // small integers: exact in bf16 and in every accumulation order
    const unsigned     m = 3, k = 4, n = 2;
    std::vector<float> A(m * k), B(k * n), want(m * n, 0.0f);
    for (unsigned i = 0; i < m * k; i++) A[i] = (float) (i % 7) - 3.0f;
    for (unsigned i = 0; i < k * n; i++) B[i] = (float) (i % 5) - 2.0f;
    for (unsigned i = 0; i < m; i++)
        for (unsigned j = 0; j < n; j++)
            for (unsigned l = 0; l < k; l++) want[i * n + j] += A[i * k + l] * B[l * n + j];
    for (int ta = 0; ta < 2; ta++)
        for (int tb = 0; tb < 2; tb++)
        {
            std::vector<uint16_t> ha(m * k), hb(k * n);
            for (unsigned i = 0; i < m; i++)
                for (unsigned l = 0; l < k; l++) ha[ta ? l * m + i : i * k + l] = bf16_of(A[i * k + l]);
            for (unsigned l = 0; l < k; l++)
                for (unsigned j = 0; j < n; j++) hb[tb ? j * k + l : l * n + j] = bf16_of(B[l * n + j]);
            MmeHip::Matrix ma(MME_HIP_BF16, ta ? k : m, ta ? m : k, ha.data(), false), mb(MME_HIP_BF16, tb ? n : k, tb ? k : n, hb.data(), false),
                my(MME_HIP_FP32, m, n);
            calculator.doGemm(my, ma, mb, ta != 0, tb != 0);
            EXPECT(std::memcmp(my.data(), want.data(), m * n * 4) == 0);
        }
    // the methods outside the path throw instead of computing
    bool thrown = false;
    try
    {
        float  v = 0.0f;
        Tensor t({1, 1, 1, 1, 1}, 2, MME_HIP_FP32, &v);
        calculator.doDma(t, t, MME_HIP_OP_AB);
    }
    catch (const MMEStackException& e)
    {
        thrown = e.status == MME_HIP_EUNSUPPORTED;
    }
    EXPECT(thrown);
    thrown = false;
    try
    {
        std::shared_ptr<Tensor> none;
        calculator.activationGemmlowp(none, none, none, none, false, MME_HIP_RM_NEAREST_EVEN, nullptr);
    }
    catch (const MMEStackException& e)
    {
        thrown = e.status == MME_HIP_EUNSUPPORTED;
    }
    EXPECT(thrown);
}

// error conventions: what MME_ASSERT rejects must throw (mme_reference_impl.cpp:465-467, 591)
static void error_conventions(Calculator& calculator)
{
    std::vector<float> a(40, 1.0f), b(40, 1.0f), y(16, 0.0f);
    bool               thrown = false;
    try
    {
        Tensor ta({5, 2, 2, 1, 1}, 3, MME_HIP_FP32, a.data()), tb({2, 5, 3, 1, 1}, 3, MME_HIP_FP32, b.data()), ty({2, 2, 3, 1, 1}, 3, MME_HIP_FP32, y.data());
        calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB); // batch 2 against batch 3
    }
    catch (const MMEStackException& e)
    {
        thrown = std::strstr(e.what(), "batch dims") != nullptr;
    }
    EXPECT(thrown);
    thrown = false;
    try
    {
        std::vector<uint16_t> y16(1, 0);
        Tensor ta({5, 1, 1, 1, 1}, 2, MME_HIP_FP32, a.data()), tb({1, 5, 1, 1, 1}, 2, MME_HIP_FP32, b.data()), ty({1, 1, 1, 1, 1}, 2, MME_HIP_BF16, y16.data());
        calculator.doBatchGemm(ty, ta, tb, MME_HIP_OP_AB); // only fp32 outputs are registered
    }
    catch (const MMEStackException& e)
    {
        thrown = std::strstr(e.what(), "not registered") != nullptr;
    }
    EXPECT(thrown);
    thrown = false;
    try
    {
        Calculator wrong(MME_HIP_CHIP_GAUDI3, 4, 4); // tensor dims must be 5
    }
    catch (const MMEStackException&)
    {
        thrown = true;
    }
    EXPECT(thrown);
}

int main()
{
    try
    {
        Calculator calculator(MME_HIP_CHIP_GAUDI3);
        struct
        {
            const char* name;
            void (*fn)(Calculator&);
        } cases[] = {{"reference_gemm_simple_test_fp32", reference_gemm_simple_test_fp32},
                     {"reference_gemm_simple_test_bf16", reference_gemm_simple_test_bf16},
                     {"reference_gemm_2d_test_fp32", reference_gemm_2d_test_fp32},
                     {"reference_gemm_2d_test_bf16", reference_gemm_2d_test_bf16},
                     {"fp8_convert", fp8_convert},
                     {"reference_gemm_simple_test_fp8", reference_gemm_simple_test_fp8},
                     {"fp16_convert_and_gemm", fp16_convert_and_gemm},
                     {"tf32_operand_clip", tf32_operand_clip},
                     {"memory_write_reductions", memory_write_reductions},
                     {"reference_gemm_api_simple_test_fp32", reference_gemm_api_simple_test_fp32},
                     {"reference_gemm_api", reference_gemm_api},
                     {"error_conventions", error_conventions}};
        for (auto& c : cases)
        {
            const int before = failures;
            c.fn(calculator);
            std::printf("%s %s\n", failures == before ? "ok    " : "FAILED", c.name);
            std::fflush(stdout);
        }
    }
    catch (const std::exception& e)
    {
        std::printf("unexpected exception: %s\n", e.what());
        return 2;
    }
    return failures ? 1 : 0;
}
