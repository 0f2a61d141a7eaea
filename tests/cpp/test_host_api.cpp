// Parity tests of the C++ operator classes (include/mm_amx_amd/kernels_gfx950.hpp) against the CPU
// oracle, written the way the reference's own drivers test amx_kernel:: (main.cpp:236-311 Matmul vs a
// naive product, :517-525 whole-N vs N-split, :884-885 MatmulVector shapes, :929 BiasGelu shape;
// weight_compression/fc16m.cpp:749-759 decode shapes; torch-ext/test.py:35-37 LinearNxN shapes).
// Needs one MI355X.  Exit status 0 = every case passed.  The oracle is linked here as the checker.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <random>
#include <thread>
#include <vector>

#include "../../include/mm_amx_amd/kernels_gfx950.hpp"
#include "../../oracle/fc_oracle.h"

using namespace gfx950_kernel;

static int g_failed = 0;
static bool throws(const std::function<void()>& f);
#define EXPECT(cond, ...)                                    \
    do {                                                     \
        if (!(cond)) {                                       \
            std::printf("    FAILED %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                        \
            std::printf("\n");                               \
            g_failed++;                                      \
        }                                                    \
    } while (0)

static std::mt19937 rng(20240229);

static std::vector<bfloat16> rand_bf16(size_t n, float stddev) {
    std::normal_distribution<float> d(0.0f, stddev);
    std::vector<bfloat16> v(n);
    for (auto& x : v) x = bfloat16(d(rng));
    return v;
}
static std::vector<int8_t> rand_i8(size_t n) {
    std::uniform_int_distribution<int> d(-127, 127);
    std::vector<int8_t> v(n);
    for (auto& x : v) x = static_cast<int8_t>(d(rng));
    return v;
}
static std::vector<float> rand_f32(size_t n, float lo, float hi) {
    std::uniform_real_distribution<float> d(lo, hi);
    std::vector<float> v(n);
    for (auto& x : v) x = d(rng);
    return v;
}
static uint16_t* bits(std::vector<bfloat16>& v) { return reinterpret_cast<uint16_t*>(v.data()); }

// relative Frobenius error and the fraction of elements within one bf16 unit in the last place
struct Err {
    double fro, within;
};
static Err compare(const std::vector<float>& got, const std::vector<float>& ref) {
    double num = 0, den = 0;
    size_t ok = 0;
    for (size_t i = 0; i < ref.size(); i++) {
        const double d = static_cast<double>(got[i]) - ref[i];
        num += d * d;
        den += static_cast<double>(ref[i]) * ref[i];
        const double a = std::fabs(static_cast<double>(ref[i]));
        const double ulp = std::exp2(std::floor(std::log2(a > 1e-37 ? a : 1e-37)) - 7);
        ok += std::fabs(d) <= ulp;
    }
    return {std::sqrt(num / (den > 0 ? den : 1)), static_cast<double>(ok) / ref.size()};
}
static std::vector<float> to_f32(const std::vector<bfloat16>& v) {
    std::vector<float> f(v.size());
    for (size_t i = 0; i < v.size(); i++) f[i] = v[i];
    return f;
}

// ---- Matmul<bf16,bf16> + BiasGeluStore<bf16, BIAS_GELU>, reference shape main.cpp:929 and friends ----
static void test_matmul_bf16_bias_gelu(int M, int K, int N, bool transB) {
    std::printf("  Matmul<bf16,bf16> BIAS_GELU M=%d K=%d N=%d transB=%d\n", M, K, N, transB);
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hB = rand_bf16(static_cast<size_t>(K) * N, 0.05f);
    auto hbias = rand_f32(N, -0.2f, 0.2f);
    tensor2D<bfloat16> A(M, K), B(transB ? N : K, transB ? K : N), C(M, N);
    tensor2D<float> Cacc(M, N);
    A.upload(hA.data());
    B.upload(hB.data());
    device_vector<float> bias(hbias);

    Matmul<bfloat16, bfloat16> mm(true, transB);
    mm(A, B, PP::BiasGeluStore<bfloat16, PP::BIAS_GELU>(C, bias.data));
    mm(A, B, PP::BiasGeluStore<float, PP::NONE>(Cacc));
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<bfloat16> got(static_cast<size_t>(M) * N);
    std::vector<float> gacc(static_cast<size_t>(M) * N);
    C.download(got.data());
    Cacc.download(gacc.data());

    std::vector<float> racc(static_cast<size_t>(M) * N);
    orc_gemm_bf16(bits(hA), K, bits(hB), transB ? K : N, transB, racc.data(), N, M, K, N, 0);
    const Err ea = compare(gacc, racc);
    EXPECT(ea.fro <= 1e-3, "accumulators: rel Frobenius %.3e", ea.fro);
    // the fused post-op equals the oracle's on the accumulators the GPU produced, bit for bit
    orc_pp pp = {};
    pp.steps = ORC_PP_BIAS | ORC_PP_GELU;
    pp.out_dtype = ORC_BF16;
    pp.bias = hbias.data();
    pp.deq_scale = 1.0f;
    std::vector<bfloat16> want(static_cast<size_t>(M) * N), ref(static_cast<size_t>(M) * N);
    orc_pp_f32(gacc.data(), N, M, N, &pp, want.data(), N * 2);
    size_t diff = 0;
    for (size_t i = 0; i < want.size(); i++) diff += want[i].bits != got[i].bits;
    EXPECT(diff == 0, "fused post-op differs from the oracle's on the same accumulators in %zu elements", diff);
    orc_pp_f32(racc.data(), N, M, N, &pp, ref.data(), N * 2);
    const Err e = compare(to_f32(got), to_f32(ref));
    EXPECT(e.fro <= 1e-3, "output: rel Frobenius %.3e", e.fro);
    // The one-ulp bar holds where the reference GELU is well conditioned: below about -3.5 its
    // 1 + x*P(x^2) cancels so far that a one-ulp change of the fp32 pre-activation moves the result by
    // more than a bf16 ulp, and MFMA does not sum in AMX's order.
    std::vector<float> g2, r2;
    for (size_t i = 0; i < ref.size(); i++)
        if (racc[i] + hbias[i % N] > -3.5f) g2.push_back(got[i]), r2.push_back(ref[i]);
    const Err ew = compare(g2, r2);
    EXPECT(ew.within >= 0.999, "output: %.3f%% within 1 bf16 ulp where GELU is well conditioned", ew.within * 100);
    EXPECT(e.within >= 0.99, "output: %.3f%% within 1 bf16 ulp over all elements", e.within * 100);
}

// ---- Matmul<int8,int8> with DEQUANT+BIAS+QUANT -> int8, bit-exact; whole N == N-split (main.cpp:517-525) ----
static void test_matmul_i8_requant(int M, int K, int N) {
    std::printf("  Matmul<s8,s8> DEQUANT|BIAS|QUANT M=%d K=%d N=%d\n", M, K, N);
    auto hA = rand_i8(static_cast<size_t>(M) * K), hB = rand_i8(static_cast<size_t>(K) * N);
    auto hbias = rand_f32(N, -0.3f, 0.3f), hq = rand_f32(N, 10.0f, 30.0f);
    tensor2D<int8_t> A(M, K), B(K, N), C(M, N), Csplit(M, N);
    tensor2D<int32_t> Cacc(M, N);
    A.upload(hA.data());
    B.upload(hB.data());
    C.zero();
    Csplit.zero();
    device_vector<float> bias(hbias), q(hq);
    constexpr PP::Steps S = static_cast<PP::Steps>(PP::DEQUANT | PP::BIAS | PP::QUANT);

    Matmul<int8_t, int8_t> mm(true, false);
    PP::BiasGeluStore<int8_t, S> pp(C, bias.data);
    pp.set_deq_scale(2e-5f);
    pp.set_q_scale(q.data);
    mm(A, B, pp);
    mm(A, B, PP::StoreI32(Cacc));
    // two column ranges, cut at a multiple of 32 as the reference's N-split does (main.cpp:461-471)
    PP::BiasGeluStore<int8_t, S> pps(Csplit, bias.data);
    pps.set_deq_scale(2e-5f);
    pps.set_q_scale(q.data);
    int cut;
    {
        int s, e;
        orc_splitter((N + 31) / 32, 2, 0, &s, &e);
        cut = e * 32;
    }
    mm(A, B, 0, cut, pps);
    mm(A, B, cut, N, pps);
    check_hip(hipDeviceSynchronize(), "sync");

    std::vector<int8_t> got(static_cast<size_t>(M) * N), gsplit(got.size()), ref(got.size());
    std::vector<int32_t> gacc(got.size()), racc(got.size());
    C.download(got.data());
    Csplit.download(gsplit.data());
    Cacc.download(gacc.data());
    orc_gemm_i8(hA.data(), K, hB.data(), N, 0, racc.data(), N, M, K, N, 0);
    orc_pp o = {};
    o.steps = ORC_PP_DEQUANT | ORC_PP_BIAS | ORC_PP_QUANT;
    o.out_dtype = ORC_I8;
    o.bias = hbias.data();
    o.deq_scale = 2e-5f;
    o.q_per_oc = hq.data();
    orc_pp_i32(racc.data(), N, M, N, &o, ref.data(), N);
    EXPECT(gacc == racc, "int32 accumulators differ");
    EXPECT(got == ref, "requantised int8 output differs");
    EXPECT(gsplit == got, "column-range split differs from the whole-N call");
    // K split over two workgroups per tile (tests/amx-mlp.cpp:560-593, 648-682): int32 partial sums add exactly
    if (K >= 1024 && M > 32) {
        tensor2D<int8_t> Ck(M, N);
        Ck.zero();
        Matmul<int8_t, int8_t> mk(true, false);
        mk.k_splits = 2;
        PP::BiasGeluStore<int8_t, S> ppk(Ck, bias.data);
        ppk.set_deq_scale(2e-5f);
        ppk.set_q_scale(q.data);
        mk(A, B, ppk);
        check_hip(hipDeviceSynchronize(), "sync");
        EXPECT(std::string(mmx_last_kernel()).find("ksplit2") != std::string::npos, "kernel %s is not a two-way K split", mmx_last_kernel());
        std::vector<int8_t> gk(got.size());
        Ck.download(gk.data());
        EXPECT(gk == ref, "two-way K split: requantised int8 output differs");
    }
}

// ---- Matmul<bf16,int8,float>: weight compression inside the op (include/kernels_amx.hpp:1319-1516) ----
static void test_matmul_weight_int8(int M, int K, int N) {
    std::printf("  Matmul<bf16,s8,f32> (weights compressed to int8) M=%d K=%d N=%d\n", M, K, N);
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hB = rand_bf16(static_cast<size_t>(K) * N, 0.05f);
    tensor2D<bfloat16> A(M, K), B(K, N);
    tensor2D<float> C(M, N);
    A.upload(hA.data());
    B.upload(hB.data());
    Matmul<bfloat16, int8_t> mm(true, false);
    mm(A, B, PP::BiasGeluStore<float, PP::DEQUANT>(C));
    if (M <= 32 && M > 16 && K >= 8192 && N <= 4096)
        EXPECT(std::string(mmx_last_kernel()).find("skinny_chunk_w8_ksplit") == 0, "ran %s, not the decode K split", mmx_last_kernel());
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<float> got(static_cast<size_t>(M) * N);
    C.download(got.data());

    std::vector<int8_t> Wq(static_cast<size_t>(K) * N);
    float qs = 0;
    const float dq = orc_quantize_weights(bits(hB), N, K, N, Wq.data(), N, &qs);
    EXPECT(dq == mm.dequant_scale_B && qs == mm.quant_scale_B, "scales: got q=%g dq=%g want q=%g dq=%g", mm.quant_scale_B,
           mm.dequant_scale_B, qs, dq);
    std::vector<float> acc(got.size()), ref(got.size());
    std::vector<float> ones(N, 1.0f);
    std::vector<uint16_t> ydummy(got.size());
    orc_gemv_w8(bits(hA), K, Wq.data(), N, 0, ones.data(), ydummy.data(), N, acc.data(), M, K, N, 0);
    for (size_t i = 0; i < ref.size(); i++) ref[i] = acc[i] * dq;
    const Err e = compare(got, ref);
    EXPECT(e.fro <= 1e-3 && e.within >= 0.999, "rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", e.fro, e.within * 100);
}

// ---- repackB_1xL<int8_t, 2>(B, scale): fc16m's own way to its int8 weights (weight_compression/fc16m.cpp:61-99, 123) ----
static void test_repack_1xL(int M, int K, int N) {
    std::printf("  repackB_1xL<int8_t,2>(B, 127/max|B|) + decode GEMM M=%d K=%d N=%d\n", M, K, N);
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hB = rand_bf16(static_cast<size_t>(K) * N, 0.05f);
    float amax = 0.0f;
    for (const auto& b : hB) amax = std::max(amax, std::fabs(static_cast<float>(b)));
    const float scale = 127.0f / amax;  // quantize_i8_scale (fc16m.cpp:113-118)
    tensor2D<bfloat16> A(M, K), B(K, N);
    tensor2D<float> C(M, N);
    A.upload(hA.data());
    B.upload(hB.data());
    PackedB<int8_t> Wp = repackB_1xL<int8_t, 2>(B, scale);
    PP::BiasGeluStore<float, PP::DEQUANT> pp(C);
    pp.set_deq_scale(1.0f / scale);
    const mmx_epilogue e = pp.descriptor();
    check(mmx_gemm(MMX_BF16, MMX_I8, A.data, A.stride, Wp.data, M, K, N, 0, N, &e, nullptr), "mmx_gemm");
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<float> got(static_cast<size_t>(M) * N);
    C.download(got.data());

    std::vector<int8_t> Wq(static_cast<size_t>(K) * N);
    orc_quantize_scale_trunc(bits(hB), N, K, N, scale, Wq.data(), N);
    std::vector<float> acc(got.size()), ref(got.size()), ones(N, 1.0f);
    std::vector<uint16_t> ydummy(got.size());
    orc_gemv_w8(bits(hA), K, Wq.data(), N, 0, ones.data(), ydummy.data(), N, acc.data(), M, K, N, 0);
    const float dq = 1.0f / scale;
    for (size_t i = 0; i < ref.size(); i++) ref[i] = acc[i] * dq;
    const Err er = compare(got, ref);
    EXPECT(er.fro <= 1e-3 && er.within >= 0.999, "rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", er.fro, er.within * 100);
    // the bf16 form is the plain pack; the preconditions are the reference's
    PackedB<bfloat16> Wb = repackB_1xL<bfloat16, 2>(B);
    EXPECT(Wb.bytes == mmx_packed_b_bytes(MMX_BF16, K, N), "bf16 form: %zu bytes", Wb.bytes);
    tensor2D<bfloat16> Bodd(K, N + 16);
    EXPECT(throws([&] { repackB_1xL<int8_t, 2>(Bodd, scale); }), "N = %d is not a multiple of 32: no error", N + 16);
}

// ---- MatmulW4: int4 weight compression inside the op (no reference counterpart beyond a timing stand-in) ----
static void test_matmul_weight_int4(int M, int K, int N) {
    std::printf("  MatmulW4 (weights compressed to int4 per output channel) M=%d K=%d N=%d\n", M, K, N);
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hB = rand_bf16(static_cast<size_t>(K) * N, 0.05f);
    tensor2D<bfloat16> A(M, K), B(K, N);
    tensor2D<float> C(M, N);
    A.upload(hA.data());
    B.upload(hB.data());
    MatmulW4 mm(true, false);
    mm(A, B, PP::BiasGeluStore<float, PP::DEQUANT>(C));
    mm(A, B, PP::BiasGeluStore<float, PP::DEQUANT>(C));  // second call: the cached packed weights
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<float> got(static_cast<size_t>(M) * N);
    C.download(got.data());

    std::vector<int8_t> q(static_cast<size_t>(K) * N);
    std::vector<float> deq(N);
    orc_quantize_int4(bits(hB), N, K, N, 0, q.data(), deq.data());
    EXPECT(mm.dequant_scales_B.to_host() == deq, "per-channel scales differ from the definition");
    std::vector<float> acc(got.size()), ref(got.size()), ones(N, 1.0f);
    std::vector<uint16_t> ydummy(got.size());
    orc_gemv_w8(bits(hA), K, q.data(), N, 0, ones.data(), ydummy.data(), N, acc.data(), M, K, N, 0);
    for (size_t i = 0; i < ref.size(); i++) ref[i] = acc[i] * deq[i % N];
    const Err e = compare(got, ref);
    EXPECT(e.fro <= 1e-3 && e.within >= 0.999, "rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", e.fro, e.within * 100);
}

// ---- MatmulVector / GemAvB, reference shapes main.cpp:884-885 ----
static void test_matvec(int M, int K) {
    std::printf("  MatmulVector / GemAvB M=%d K=%d\n", M, K);
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hb = rand_bf16(K, 1.0f);
    tensor2D<bfloat16> A(M, K);
    A.upload(hA.data());
    device_vector<bfloat16> b(hb);
    device_vector<float> c(M), c2(M);
    MatmulVector<bfloat16, bfloat16>()(A, b.data, c.data);
    GemAvB()(A, b.data, c2.data);
    std::vector<float> ref(M), ref2(M);
    orc_matvec_bf16(bits(hA), K, bits(hb), ref.data(), M, K);
    orc_gemavb_bf16(bits(hA), K, bits(hb), ref2.data(), M, K);
    const Err e = compare(c.to_host(), ref), e2 = compare(c2.to_host(), ref2);
    EXPECT(e.fro <= 1e-5, "MatmulVector bf16 rel Frobenius %.3e", e.fro);
    EXPECT(e2.fro <= 1e-5, "GemAvB rel Frobenius %.3e", e2.fro);

    auto hAi = rand_i8(static_cast<size_t>(M) * K), hbi = rand_i8(K);
    tensor2D<int8_t> Ai(M, K);
    Ai.upload(hAi.data());
    device_vector<int8_t> bi(hbi);
    device_vector<int32_t> ci(M);
    MatmulVector<int8_t, int8_t>()(Ai, bi.data, ci.data);
    std::vector<int32_t> refi(M);
    orc_matvec_i8(hAi.data(), K, hbi.data(), refi.data(), M, K);
    EXPECT(ci.to_host() == refi, "MatmulVector int8 differs");
}

// ---- the unsigned byte forms (include/kernels_amx.hpp:839-850, 1057-1101) ----
template <typename TA, typename TB>
static void test_unsigned_bytes(int M, int K, int N) {
    std::printf("  Matmul / MatmulVector <%s8,%s8> M=%d K=%d N=%d\n", std::is_same<TA, uint8_t>::value ? "u" : "s",
                std::is_same<TB, uint8_t>::value ? "u" : "s", M, K, N);
    auto rA = rand_i8(static_cast<size_t>(M) * K), rB = rand_i8(static_cast<size_t>(K) * N);  // any byte pattern
    tensor2D<TA> A(M, K);
    tensor2D<TB> B(K, N);
    tensor2D<int32_t> C(M, N);
    A.upload(reinterpret_cast<const TA*>(rA.data()));
    B.upload(reinterpret_cast<const TB*>(rB.data()));
    Matmul<TA, TB> mm(true, false);
    mm(A, B, PP::StoreI32(C));
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<int32_t> got(static_cast<size_t>(M) * N), ref(got.size());
    C.download(got.data());
    orc_gemm_x8(std::is_same<TA, uint8_t>::value, std::is_same<TB, uint8_t>::value, rA.data(), K, rB.data(), N, 0, ref.data(), N, M, K, N);
    EXPECT(got == ref, "unsigned-byte Matmul differs from the integer product");
    device_vector<TB> b(std::vector<TB>(reinterpret_cast<const TB*>(rB.data()), reinterpret_cast<const TB*>(rB.data()) + K));
    device_vector<int32_t> c(M);
    MatmulVector<TA, TB>()(A, b.data, c.data);
    std::vector<int32_t> refv(M);
    orc_matvec_x8(std::is_same<TA, uint8_t>::value, std::is_same<TB, uint8_t>::value, rA.data(), K, rB.data(), refv.data(), M, K);
    EXPECT(c.to_host() == refv, "unsigned-byte MatmulVector differs from the integer product");
}

// ---- LinearNxN call shape (torch-ext/test.py:35-37, 108-119) ----
static void test_linear_nxn(int M, int K, int N) {
    std::printf("  LinearNxN M=%d K=%d N=%d\n", M, K, N);
    auto hx = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hw = rand_bf16(static_cast<size_t>(N) * K, 0.05f);
    tensor2D<bfloat16> x(M, K), w(N, K);
    tensor2D<float> y(M, N), y2(M, N);
    x.upload(hx.data());
    w.upload(hw.data());
    LinearNxN lin;
    lin.set_weight(w);
    lin.forward(x, y);
    LinearNxN copy = lin.deepcopy();
    copy.forward(x, y2);
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<float> got(static_cast<size_t>(M) * N), got2(got.size()), ref(got.size());
    y.download(got.data());
    y2.download(got2.data());
    orc_gemm_bf16(bits(hx), K, bits(hw), K, 1, ref.data(), N, M, K, N, 0);
    const Err e = compare(got, ref);
    EXPECT(e.fro <= 1e-3 && e.within >= 0.999, "rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", e.fro, e.within * 100);
    EXPECT(got == got2, "deep copy gives a different result");
}

// ---- MLP, stage by stage (h from the same x; y from the same h) ----
static void test_mlp(int M, int K, int N, int down_k_splits = 0) {
    std::printf("  MLP M=%d K=%d N=%d down_k_splits=%d\n", M, K, N, down_k_splits);
    auto hx = rand_bf16(static_cast<size_t>(M) * K, 1.0f);
    auto hg = rand_bf16(static_cast<size_t>(N) * K, 0.02f), hu = rand_bf16(static_cast<size_t>(N) * K, 0.02f);
    auto hd = rand_bf16(static_cast<size_t>(K) * N, 0.02f);
    tensor2D<bfloat16> x(M, K), wg(N, K), wu(N, K), wd(K, N), y(M, K);
    x.upload(hx.data());
    wg.upload(hg.data());
    wu.upload(hu.data());
    wd.upload(hd.data());
    MLP mlp;
    mlp.down_k_splits = down_k_splits;
    mlp.setup(wg, wu, wd);
    mlp.run(x, y);
    if (down_k_splits > 1 || (M <= 32 && M > 8 && N >= 8192))  // (few panels of a long K at decode sizes: the library's own split)
        EXPECT(std::string(mmx_last_kernel()).find("ksplit") != std::string::npos, "down projection ran %s, not a K split", mmx_last_kernel());
    check_hip(hipDeviceSynchronize(), "sync");
    std::vector<bfloat16> gh(static_cast<size_t>(M) * N), gy(static_cast<size_t>(M) * K);
    tensor2D<bfloat16> hview(M, N, mlp.actUp.data, mlp.actUp.stride);
    hview.download(gh.data());
    y.download(gy.data());

    std::vector<bfloat16> rh(gh.size()), ry(gy.size()), ry_from_gh(gy.size());
    orc_mlp(bits(hx), bits(hg), bits(hu), bits(hd), bits(rh), bits(ry), M, K, N, 0, 0);
    const Err eh = compare(to_f32(gh), to_f32(rh));
    EXPECT(eh.fro <= 1e-3 && eh.within >= 0.999, "h: rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", eh.fro, eh.within * 100);
    orc_mlp_down(bits(gh), bits(hd), bits(ry_from_gh), M, K, N, down_k_splits == 2 ? 1 : 0, 0);
    const Err ey = compare(to_f32(gy), to_f32(ry_from_gh));
    EXPECT(ey.fro <= 1e-3 && ey.within >= 0.999, "y from the GPU's h: rel Frobenius %.3e, %.3f%% within 1 bf16 ulp", ey.fro,
           ey.within * 100);
    const Err ee = compare(to_f32(gy), to_f32(ry));
    EXPECT(ee.fro <= 1e-3, "y end to end: rel Frobenius %.3e", ee.fro);
}

// ---- first calls from two threads at once: nothing in the library may race on its one-time set-up, and the tuning
// knobs of one thread must not reach the other ----
static void test_two_threads_first_call() {
    std::printf("  first calls from two threads\n");
    const int M = 300, K = 256, N = 512;
    auto hA = rand_bf16(static_cast<size_t>(M) * K, 1.0f), hB = rand_bf16(static_cast<size_t>(K) * N, 0.05f);
    std::vector<float> racc(static_cast<size_t>(M) * N);
    orc_gemm_bf16(bits(hA), K, bits(hB), N, 0, racc.data(), N, M, K, N, 0);
    std::vector<float> got[2];
    std::string kernels[2], errors[2];
    const char* tiles[2] = {"256x256", "128x256"};  // kernel variants no earlier test has launched with fp32 outputs
    auto worker = [&](int t) {
        try {
            check_hip(hipSetDevice(0), "hipSetDevice");
            check(mmx_set_tile(tiles[t]), "mmx_set_tile");
            hipStream_t st;
            check_hip(hipStreamCreate(&st), "hipStreamCreate");
            tensor2D<bfloat16> A(M, K), B(K, N);
            tensor2D<float> C(M, N);
            A.upload(hA.data());
            B.upload(hB.data());
            Matmul<bfloat16, bfloat16> mm(true, false);
            for (int rep = 0; rep < 3; rep++) mm(A, B, PP::BiasGeluStore<float, PP::NONE>(C), st);
            kernels[t] = mmx_last_kernel();
            check_hip(hipStreamSynchronize(st), "sync");
            got[t].resize(racc.size());
            C.download(got[t].data());
            check_hip(hipStreamDestroy(st), "hipStreamDestroy");
        } catch (const std::exception& e) {
            errors[t] = e.what();
        }
    };
    std::thread t0(worker, 0), t1(worker, 1);
    t0.join();
    t1.join();
    for (int t = 0; t < 2; t++) {
        EXPECT(errors[t].empty(), "thread %d: %s", t, errors[t].c_str());
        EXPECT(kernels[t].find(tiles[t]) != std::string::npos, "thread %d ran %s, its own tile choice was %s", t, kernels[t].c_str(), tiles[t]);
        if (!got[t].empty()) {
            const Err e = compare(got[t], racc);
            EXPECT(e.fro <= 1e-3 && e.within >= 0.999, "thread %d: rel Frobenius %.3e", t, e.fro);
        }
    }
}

// ---- preconditions raise where the reference asserts ----
static bool throws(const std::function<void()>& f) {
    try {
        f();
    } catch (const std::runtime_error&) {
        return true;
    }
    return false;
}
static void test_errors() {
    std::printf("  preconditions\n");
    tensor2D<bfloat16> A(4, 16), B(16, 32), C(4, 32);
    Matmul<bfloat16, bfloat16> mm;
    EXPECT(throws([&] { mm(A, B, PP::BiasGeluStore<bfloat16, PP::NONE>(C)); }), "K < kStep must throw");
    PP::BiasGeluStore<bfloat16, PP::NONE> pp(C);
    EXPECT(throws([&] { pp.set_bias(nullptr); }), "set_bias without BIAS must throw");
    EXPECT(throws([&] { pp.set_deq_scale(2.0f); }), "set_deq_scale without DEQUANT must throw");
    EXPECT(throws([&] { pp.set_q_scale(2.0f); }), "set_q_scale without QUANT must throw");
    tensor2D<bfloat16> w(48, 40);
    LinearNxN lin;
    EXPECT(throws([&] { lin.set_weight(w); }), "set_weight with N, K not multiples of 32 must throw");
    tensor2D<bfloat16> A2(4, 64), B2(32, 32);
    EXPECT(throws([&] { mm(A2, B2, PP::BiasGeluStore<bfloat16, PP::NONE>(C)); }), "mismatched K must throw");
}

int main() {
    try {
        init(0);
        std::printf("oracle hot loop: %s\n", orc_isa());
        test_matmul_bf16_bias_gelu(88, 77, 66, false);   // main.cpp:929
        test_matmul_bf16_bias_gelu(735, 337, 271, true);  // main.cpp:733, M, K and N tails
        test_matmul_bf16_bias_gelu(512, 1024, 768, false);
        test_matmul_i8_requant(256, 512, 320);
        test_matmul_i8_requant(77, 200, 95);
        test_matmul_weight_int8(2, 2560, 192);  // fc16m.cpp:749
        test_matmul_weight_int8(160, 512, 256);   // large M: int8 fragments converted between LDS and the MFMA operand
        test_matmul_weight_int8(300, 200, 96);    // ... with a K tail (masked loads)
        test_matmul_weight_int8(24, 8192, 256);   // decode with few panels: K walked in slices through the stream's workspace
        test_repack_1xL(2, 2560, 192);            // fc16m.cpp:749
        test_repack_1xL(16, 512, 352);
        test_matmul_weight_int4(1, 4096, 352);
        test_matmul_weight_int4(7, 300, 77);
        test_matvec(901, 80);  // main.cpp:884
        test_matvec(901, 96);  // main.cpp:885
        test_unsigned_bytes<uint8_t, int8_t>(77, 200, 95);
        test_unsigned_bytes<int8_t, uint8_t>(160, 512, 96);
        test_unsigned_bytes<uint8_t, uint8_t>(16, 4096, 64);
        test_linear_nxn(32, 32, 32);  // torch-ext/test.py:35
        test_linear_nxn(512, 128, 4096);  // torch-ext/test.py:37
        test_mlp(1, 512, 1024);
        test_mlp(96, 512, 1024);
        test_mlp(24, 512, 8192);    // decode: the down projection (K = 8192, 16 panels) takes its own K split
        test_mlp(96, 512, 1024, 2);  // the reference's do_splitK for the down projection (tests/amx-mlp.cpp:768)
        test_matmul_i8_requant(160, 2048, 320);  // long enough K for the two-way K split
        test_two_threads_first_call();
        test_errors();
    } catch (const std::exception& e) {
        std::printf("EXCEPTION: %s\n", e.what());
        return 2;
    }
    std::printf(g_failed ? "%d check(s) FAILED\n" : "all checks passed\n", g_failed);
    return g_failed ? 1 : 0;
}
