// The reference's own classes -- MmeSimTensor, Matrix, ConvolutionParams and CPUCalculator, from the headers of
// mme/mme_reference -- with CPUCalculator's methods supplied by include/reference_stub/mme_reference_hip.cpp instead of
// mme_reference_impl.cpp: what a caller of the reference runs after the switch.  Built by oracle/Makefile (target
// ref_dropin) from the reference's tensor sources where they lie, the stub and this file; run by
// tests/test_gpu_cpp_kat.py on a GPU.  Expected values are closed forms and what the genuine reference calculator computes on
// the same tensor objects (tests/cpp/dropin_reference_side.cpp: the reference's class compiled under another name).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
#include <vector>

#include "convolution_params.h"
#include "mme_reference.h"
#include "sim_tensor.h"

using namespace MmeCommon;

void reference_side_batch_gemm(MmeSimTensor& y, const MmeSimTensor& a, const MmeSimTensor& b, EMmeOpType op);
void reference_side_convolution(MmeSimTensor& out, const MmeSimTensor& x, const MmeSimTensor& w, const MmeSimTensor& y, const ConvolutionParams& p, EMmeOpType op);
void reference_side_activation(pMMESimTensor out, const pMMESimTensor acc, bool relu, RoundingMode rm, bool clipFp);

static double rel_frobenius(const float* got, const float* want, size_t n)
{
    double num = 0, den = 0;
    for (size_t i = 0; i < n; i++)
    {
        const double d = (double) got[i] - want[i];
        num += d * d;
        den += (double) want[i] * want[i];
    }
    return std::sqrt(num / (den > 0 ? den : 1));
}

static int failures = 0;
static void check(bool ok, const char* name)
{
    std::printf("%s %s\n", ok ? "ok" : "FAILED", name);
    if (!ok) failures++;
}

static uint16_t to_bf16(float x)
{
    uint32_t u;
    std::memcpy(&u, &x, 4);
    return (uint16_t) ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static float from_bf16(uint16_t h)
{
    const uint32_t u = (uint32_t) h << 16;
    float          x;
    std::memcpy(&x, &u, 4);
    return x;
}

int main()
{
    CPUCalculator calc(e_mme_Gaudi3, 5, 4);

    // a dot product of five tens, through doBatchGemm on tensors and through doGemm on matrices
    {
        SizeArray as = {5, 1, 1, 1, 1}, bs = {1, 5, 1, 1, 1}, ys = {1, 1, 1, 1, 1};
        MmeSimTensor a(as, 2, e_type_fp32), b(bs, 2, e_type_fp32), y(ys, 2, e_type_fp32);
        for (int i = 0; i < 5; i++) ((float*) a.data())[i] = ((float*) b.data())[i] = 10.0f;
        calc.doBatchGemm(y, a, b, e_mme_ab);
        check(*(float*) y.data() == 500.0f, "doBatchGemm on the reference's MmeSimTensor: 5 x 10 * 10 = 500");

        Matrix ma(e_type_fp32, 1, 5), mb(e_type_fp32, 5, 1), my(e_type_fp32, 1, 1);
        for (int i = 0; i < 5; i++) ((float*) ma.data())[i] = ((float*) mb.data())[i] = 10.0f;
        calc.doGemm(my, ma, mb, false, false);
        check(*(float*) my.data() == 500.0f, "doGemm on the reference's Matrix: 500");
    }

    // bf16 GEMM, 96 x 72 times 72 x 80, against sums in double precision of the same bf16 values
    {
        const int    M = 96, K = 72, N = 80;
        SizeArray    as = {(unsigned) K, (unsigned) M, 1, 1, 1}, bs = {(unsigned) N, (unsigned) K, 1, 1, 1}, ys = {(unsigned) N, (unsigned) M, 1, 1, 1};
        MmeSimTensor a(as, 2, e_type_bf16), b(bs, 2, e_type_bf16), y(ys, 2, e_type_fp32);
        std::mt19937 gen(7);
        std::normal_distribution<float> dist(0.0f, 1.0f);
        uint16_t *pa = (uint16_t*) a.data(), *pb = (uint16_t*) b.data();
        for (int i = 0; i < M * K; i++) pa[i] = to_bf16(dist(gen));
        for (int i = 0; i < K * N; i++) pb[i] = to_bf16(dist(gen));
        calc.doBatchGemm(y, a, b, e_mme_ab);
        MmeSimTensor yr(ys, 2, e_type_fp32);
        reference_side_batch_gemm(yr, a, b, e_mme_ab);
        check(rel_frobenius((float*) y.data(), (float*) yr.data(), (size_t) M * N) <= 2e-3,
              "bf16 GEMM 96 x 72 x 80 on MmeSimTensor within 2e-3 of the reference calculator's on the same tensors");
        MmeSimTensor yt(ys, 2, e_type_fp32), ytr(ys, 2, e_type_fp32);
        SizeArray    ats = {(unsigned) M, (unsigned) K, 1, 1, 1};
        MmeSimTensor at(ats, 2, e_type_bf16);
        for (int m = 0; m < M; m++)
            for (int k = 0; k < K; k++) ((uint16_t*) at.data())[k * M + m] = pa[m * K + k];
        calc.doBatchGemm(yt, at, b, e_mme_atb);
        reference_side_batch_gemm(ytr, at, b, e_mme_atb);
        check(rel_frobenius((float*) yt.data(), (float*) ytr.data(), (size_t) M * N) <= 2e-3 &&
                  rel_frobenius((float*) yt.data(), (float*) y.data(), (size_t) M * N) <= 1e-6,
              "the same product with A stored K x M (atb): within 2e-3 of the reference, equal to the ab result");
    }

    // 3 x 3 forward convolution, bf16, 2 images of 6 x 5 pixels, 16 -> 32 channels, padding 1, against a direct sum
    {
        const int    C = 16, Kc = 32, W = 6, H = 5, B = 2;
        SizeArray    xs = {(unsigned) C, (unsigned) W, (unsigned) H, 1, (unsigned) B}, ws = {(unsigned) Kc, (unsigned) C, 3, 3, 1},
                  ys = {(unsigned) Kc, (unsigned) W, (unsigned) H, 1, (unsigned) B};
        MmeSimTensor x(xs, 5, e_type_bf16), w(ws, 5, e_type_bf16), y(ys, 5, e_type_fp32);
        std::mt19937 gen(11);
        std::normal_distribution<float> dist(0.0f, 1.0f);
        uint16_t *px = (uint16_t*) x.data(), *pw = (uint16_t*) w.data();
        for (int i = 0; i < C * W * H * B; i++) px[i] = to_bf16(dist(gen));
        for (int i = 0; i < Kc * C * 9; i++) pw[i] = to_bf16(0.3f * dist(gen));
        ConvolutionParams p;
        p.dim = 2;
        for (int d = 0; d < 3; d++)
        {
            p.padding[d] = d < 2 ? 1 : 0;
            p.convStride[d] = 1;
            p.dilation[d] = 1;
        }
        calc.doConvolution(y, x, w, y, p, e_mme_fwd);
        MmeSimTensor yr(ys, 5, e_type_fp32);
        reference_side_convolution(yr, x, w, yr, p, e_mme_fwd);
        check(rel_frobenius((float*) y.data(), (float*) yr.data(), (size_t) Kc * W * H * B) <= 2e-3,
              "bf16 3 x 3 forward convolution on MmeSimTensor within 2e-3 of the reference calculator's");
        // dedx and dedw of the same layer with y as the gradient
        MmeSimTensor g(ys, 5, e_type_bf16), dx(xs, 5, e_type_fp32), dxr(xs, 5, e_type_fp32), dw(ws, 5, e_type_fp32), dwr(ws, 5, e_type_fp32);
        for (int i = 0; i < Kc * W * H * B; i++) ((uint16_t*) g.data())[i] = to_bf16(0.5f * dist(gen));
        calc.doConvolution(dx, x, w, g, p, e_mme_dedx);
        reference_side_convolution(dxr, x, w, g, p, e_mme_dedx);
        calc.doConvolution(dw, x, w, g, p, e_mme_dedw);
        reference_side_convolution(dwr, x, w, g, p, e_mme_dedw);
        check(rel_frobenius((float*) dx.data(), (float*) dxr.data(), (size_t) C * W * H * B) <= 2e-3 &&
                  rel_frobenius((float*) dw.data(), (float*) dwr.data(), (size_t) Kc * C * 9) <= 2e-3,
              "dedx and dedw of the same layer within 2e-3 of the reference calculator's");
    }

    // doActivation: fp32 accumulators to bf16 with relu, round to nearest even
    {
        SizeArray  s = {8, 1, 1, 1, 1};
        auto       acc = std::make_shared<MmeSimTensor>(s, 2, e_type_fp32), out = std::make_shared<MmeSimTensor>(s, 2, e_type_bf16);
        const float in[8] = {1.0f, -2.0f, 0.5f, 3.0f + 1.0f / 256, 1e-3f, -0.0f, 65536.0f, 1.0f + 3.0f / 256};
        std::memcpy(acc->data(), in, sizeof in);
        calc.doActivation(out, acc, nullptr, nullptr, true);
        bool ok = true;
        for (int i = 0; i < 8; i++) ok = ok && ((uint16_t*) out->data())[i] == to_bf16(in[i] > 0 ? in[i] : 0.0f);
        check(ok, "doActivation with relu on shared_ptr<MmeSimTensor>: bf16 codes equal round-to-nearest-even of max(x, 0)");
        SizeArray   s8 = {4096, 1, 1, 1, 1};
        auto        acc8 = std::make_shared<MmeSimTensor>(s8, 2, e_type_fp32);
        auto        o8 = std::make_shared<MmeSimTensor>(s8, 2, e_type_fp8_143, nullptr, 7), o8r = std::make_shared<MmeSimTensor>(s8, 2, e_type_fp8_143, nullptr, 7);
        std::mt19937 gen(3);
        std::normal_distribution<float> dist(0.0f, 40.0f);
        for (int i = 0; i < 4096; i++) ((float*) acc8->data())[i] = dist(gen) * (i % 7 == 0 ? 20.0f : 1.0f);
        calc.doActivation(o8, acc8, nullptr, nullptr, false, RoundToNearest, nullptr, true);
        reference_side_activation(o8r, acc8, false, RoundToNearest, true);
        check(std::memcmp(o8->data(), o8r->data(), 4096) == 0, "doActivation to fp8_143 (bias 7, clipping): every code equal to the reference calculator's");
    }

    // what the Gaudi3 flow never reaches throws
    {
        bool threw = false;
        try
        {
            calc.activationGemmlowp(nullptr, nullptr, nullptr, nullptr, false, RoundToNearest, nullptr);
        }
        catch (const std::exception&)
        {
            threw = true;
        }
        check(threw, "activationGemmlowp throws");
    }
    std::printf(failures ? "%d FAILED\n" : "all ok\n", failures);
    return failures ? 1 : 0;
}
