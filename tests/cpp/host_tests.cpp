// Tests of the host-side TFCC layer, modelled on the reference's own gtest cases:
//   framework  tfcc/test/framework.cpp:37-171   (reshape, expand_dims, squeeze, FlexAllocator accounting)
//   data       tfcc/test/data.cpp:34-72
//   blas       tfcc/test/blas.cpp:34-61          (four shape families, with and without bias)
//   quantization tfcc/test/quantization.cpp:62-218 (known answers, 5/11/17 round trips, exact int32)
// usage: host_tests cpu | gpu      ("cpu" needs no GPU: host-memory device, no compute interfaces)
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <algorithm>
#include <array>
#include <random>
#include <string>
#include <thread>

#include "tfcc_layers.h"
#include "tfcc_rocm_device.h"

static int g_failures = 0;
static int g_checks = 0;

#define CHECK(cond)                                                                  \
  do {                                                                               \
    ++g_checks;                                                                      \
    if (!(cond)) {                                                                   \
      ++g_failures;                                                                  \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                \
    }                                                                                \
  } while (0)

#define CHECK_THROWS(expr, TYPE)                                                     \
  do {                                                                               \
    ++g_checks;                                                                      \
    bool caught = false;                                                             \
    try {                                                                            \
      (void)(expr);                                                                  \
    } catch (const TYPE&) {                                                          \
      caught = true;                                                                 \
    } catch (...) {                                                                  \
    }                                                                                \
    if (!caught) {                                                                   \
      ++g_failures;                                                                  \
      std::printf("  FAILED %s:%d: %s did not throw %s\n", __FILE__, __LINE__, #expr, #TYPE); \
    }                                                                                \
  } while (0)

#define CHECK_THROWS_MSG(expr, TYPE, TEXT)                                           \
  do {                                                                               \
    ++g_checks;                                                                      \
    bool caught = false;                                                             \
    try {                                                                            \
      (void)(expr);                                                                  \
    } catch (const TYPE& e) {                                                        \
      caught = std::string(e.what()) == (TEXT);                                      \
      if (!caught) std::printf("  message was: %s\n", e.what());                     \
    } catch (...) {                                                                  \
    }                                                                                \
    if (!caught) {                                                                   \
      ++g_failures;                                                                  \
      std::printf("  FAILED %s:%d: %s did not throw %s(\"%s\")\n", __FILE__, __LINE__, #expr, #TYPE, TEXT); \
    }                                                                                \
  } while (0)

static void run(const char* name, const std::function<void()>& body) {
  int before = g_failures;
  std::printf("[ RUN  ] %s\n", name);
  std::fflush(stdout);
  try {
    body();
  } catch (const std::exception& e) {
    ++g_failures;
    std::printf("  FAILED: unexpected exception: %s\n", e.what());
  }
  std::printf("[ %s ] %s\n", g_failures == before ? " OK " : "FAIL", name);
  std::fflush(stdout);
}

// ---- framework (any device) ---------------------------------------------------------------------------

static void test_reshape() {
  tfcc::Variable<float> expect({3, 4, 5});
  tfcc::Variable<float> a({60});
  tfcc::View<float> b(a);
  a.reshape({3, 4, 5});
  b.reshape({3, 4, 5});
  CHECK(a.shape() == expect.shape());
  CHECK(b.shape() == expect.shape());
  CHECK_THROWS_MSG(a.reshape({4, 4, 4}), tfcc::InvalidArgumentError, "shape area couldn't be changed");
  CHECK_THROWS(b.reshape({4, 4, 4}), tfcc::InvalidArgumentError);
}

static void test_expand_dims() {
  tfcc::Variable<float> expect({3, 1, 4, 5});
  tfcc::Variable<float> a({3, 4, 5});
  tfcc::View<float> b(a);
  a.expandDims(1);
  b.expandDims(1);
  CHECK(a.shape() == expect.shape());
  CHECK(b.shape() == expect.shape());
  CHECK_THROWS(a.expandDims(5), tfcc::InvalidArgumentError);
  CHECK_THROWS(b.expandDims(5), tfcc::InvalidArgumentError);
}

static void test_squeeze() {
  {
    tfcc::Variable<float> expect({3, 4, 5});
    tfcc::Variable<float> a({3, 1, 4, 1, 5, 1});
    tfcc::View<float> b(a);
    a.squeeze();
    b.squeeze();
    CHECK(a.shape() == expect.shape());
    CHECK(b.shape() == expect.shape());
  }
  {
    tfcc::Variable<float> expect({3, 1, 4, 5});
    tfcc::Variable<float> a({3, 1, 4, 1, 5, 1});
    tfcc::View<float> b(a);
    a.squeeze({3, 5});
    b.squeeze({3, 5});
    CHECK(a.shape() == expect.shape());
    CHECK(b.shape() == expect.shape());
    CHECK_THROWS(a.squeeze({4}), tfcc::InvalidArgumentError);
    CHECK_THROWS(b.squeeze({4}), tfcc::InvalidArgumentError);
    CHECK_THROWS(a.squeeze({0}), tfcc::InvalidArgumentError);
    CHECK_THROWS(b.squeeze({0}), tfcc::InvalidArgumentError);
  }
}

static void test_view_window() {
  tfcc::Variable<float> a({6, 4});
  tfcc::View<float> whole(a);
  CHECK(whole.data() == a.data() && whole.shape() == a.shape());
  tfcc::View<float> tail(a, tfcc::Shape({3, 8}), 1);
  CHECK(tail.shape() == tfcc::Shape({2, 8}) && tail.data() == a.data() + 8);
  tfcc::View<float> mid(a, a.shape(), 2, 5);
  CHECK(mid.shape() == tfcc::Shape({3, 4}) && mid.data() == a.data() + 8);
  tfcc::View<float> clipped(a, a.shape(), 4, 100);
  CHECK(clipped.shape() == tfcc::Shape({2, 4}));
  CHECK_THROWS_MSG(tfcc::View<float>(a, tfcc::Shape({5, 5})), tfcc::InvalidArgumentError, "invalid shape");
  CHECK_THROWS_MSG(tfcc::View<float>(a, a.shape(), 6), tfcc::InvalidArgumentError, "invalid start");
}

static void test_flexallocator() {
  auto* allocator = dynamic_cast<tfcc::FlexAllocator*>(&tfcc::Session::getThreadDefault()->getAllocator());
  CHECK(allocator != nullptr);
  if (!allocator) return;
  allocator->releaseCache();
  CHECK(allocator->used() == 0);
  const unsigned block = 1024 - 64 / sizeof(float);  // one 4 KiB bucket including the 64-byte header
  allocator->setLimit(4096 * 8);
  {
    tfcc::Variable<float> x1({block}), x2({block}), x3({block}), x4({block}), x5({block}), x6({block}), x7({block}),
        x8({block});
    CHECK_THROWS(tfcc::Variable<float>({64}), tfcc::ResourceExhaustedError);
  }
  allocator->releaseCache();
  CHECK(allocator->used() == 0);

  allocator->setFlexLimit(4096 * 4);
  {
    tfcc::Variable<float> x;
    x = tfcc::Variable<float>({block});
    CHECK(allocator->used() == 4096u);
    x = tfcc::Variable<float>({2, block});
    CHECK(allocator->used() == 4096u * 3);
    x = tfcc::Variable<float>({3, block});
    CHECK(allocator->used() == 4096u * 5);
    x = tfcc::Variable<float>({3, block});
    CHECK(allocator->used() == 4096u * 6);
    tfcc::Variable<float> x2({4, block});
    CHECK(allocator->used() == 4096u * 7);
  }
  allocator->releaseCache();
  CHECK(allocator->used() == 0);
  allocator->setFlexLimit(4096 * 4 - 1);
  {
    tfcc::Variable<float> x;
    x = tfcc::Variable<float>({block});
    CHECK(allocator->used() == 4096u);
    x = tfcc::Variable<float>({2, block});
    CHECK(allocator->used() == 4096u * 3);
    x = tfcc::Variable<float>();
    x = tfcc::Variable<float>({3, block});
    CHECK(allocator->used() == 4096u * 3);
  }
  allocator->setFlexLimit(0);
  allocator->setLimit(0);
  allocator->releaseCache();
}

static void test_matmul_validation() {
  // tfcc/core/operations/tfcc_blas.cpp:26-54: thrown before any device work
  using tfcc::InvalidArgumentError;
  tfcc::Variable<float> v3({3}), m34({3, 4}), m45({4, 5}), m56({5, 6}), b234({2, 3, 4}), b5647({5, 6, 4, 7}),
      b345({3, 4, 5}), bias4({4}), bias15({1, 5});
  CHECK_THROWS_MSG(tfcc::blas::matmul(v3, m34), InvalidArgumentError, "matmul require tensors with two or more dimensions");
  CHECK_THROWS_MSG(tfcc::blas::matmul(b234, b5647), InvalidArgumentError, "shape invalid");
  CHECK_THROWS_MSG(tfcc::blas::matmul(m34, m56), InvalidArgumentError, "shape invalid");
  CHECK_THROWS_MSG(tfcc::blas::matmul(b234, b345), InvalidArgumentError, "shape invalid");  // unequal leading dimensions
  CHECK_THROWS_MSG(tfcc::blas::matmul(m34, m45, bias4), InvalidArgumentError, "shape invalid");
  CHECK_THROWS_MSG(tfcc::blas::matmul(m34, m45, bias15), InvalidArgumentError, "shape invalid");
  tfcc::Variable<float> e({2, 0, 4}), f({2, 4, 5});
  tfcc::Variable<float> r = tfcc::blas::matmul(e, f);  // empty operand: result shape only
  CHECK(r.shape() == tfcc::Shape({2, 0, 5}) && r.size() == 0);
  tfcc::Variable<double> da({3, 4}), db({4, 5});
  CHECK_THROWS(tfcc::blas::matmul(da, db), tfcc::NotImplementedError);  // only float has a blas backend
}

static void test_device_identity(tfcc::DeviceType expected) {
  tfcc::Device* d = tfcc::Device::getThreadDefault();
  CHECK(d != nullptr);
  CHECK(d->getDeviceType() == expected);
  CHECK((d->getDeviceID() >> 24) == static_cast<unsigned>(expected));
}

// ---- GPU --------------------------------------------------------------------------------------------

static void test_data() {
  // tfcc/test/data.cpp:34-72
  std::vector<float> values(3 * 4 * 5);
  for (size_t i = 0; i < values.size(); ++i) values[i] = static_cast<float>(i) * 0.5f - 7;
  tfcc::Variable<float> a({3, 4, 5});
  tfcc::data::set(a, values);
  CHECK(tfcc::data::get(a) == values);
  tfcc::View<float> tail(a, a.shape(), 1);
  std::vector<float> got = tfcc::data::get(tail);
  CHECK(got.size() == 40 && got[0] == values[20] && got[39] == values[59]);
  tfcc::Variable<float> c = tfcc::data::copy(a);
  CHECK(tfcc::data::get(c) == values);
  tfcc::data::zeros(c);
  for (float v : tfcc::data::get(c)) CHECK(v == 0.f);
  tfcc::Variable<int32_t> o({7});
  tfcc::data::ones(o);
  for (int32_t v : tfcc::data::get(o)) CHECK(v == 1);
  tfcc::Variable<uint8_t> u = tfcc::data::set(std::vector<uint8_t>{1, 2, 255}, {3});
  CHECK((tfcc::data::get(u) == std::vector<uint8_t>{1, 2, 255}));
  CHECK_THROWS(tfcc::data::set(a, std::vector<float>(5)), tfcc::InvalidArgumentError);
}

static bool is_similar(float x, float y) {
  // tfcc/core/utils/tfcc_debugutils.cpp:102-111
  return std::fabs(x - y) < 1e-3f * std::fabs(x + y) || std::fabs(x - y) < 1e-5f;
}

static void matmul_case(std::mt19937& rng, const std::vector<unsigned>& sa, const std::vector<unsigned>& sb) {
  std::uniform_real_distribution<float> dist(-1.f, 1.f);
  tfcc::Shape shapeA(sa), shapeB(sb);
  std::vector<float> ha(shapeA.area()), hb(shapeB.area());
  for (auto& v : ha) v = dist(rng);
  for (auto& v : hb) v = dist(rng);
  const unsigned m = sa[sa.size() - 2], k = sa.back(), n = sb.back();
  std::vector<float> hbias(n);
  for (auto& v : hbias) v = dist(rng);
  tfcc::Variable<float> a = tfcc::data::set(ha, shapeA), b = tfcc::data::set(hb, shapeB), bias = tfcc::data::set(hbias, {n});
  tfcc::Variable<float> r = tfcc::blas::matmul(a, b), rb = tfcc::blas::matmul(a, b, bias);
  std::vector<unsigned> expectShape = sa.size() > sb.size() ? sa : sb;
  expectShape[expectShape.size() - 2] = m;
  expectShape[expectShape.size() - 1] = n;
  CHECK(r.shape() == tfcc::Shape(expectShape) && rb.shape() == tfcc::Shape(expectShape));
  const unsigned batch = r.size() / (m * n);
  const size_t strideA = sa.size() == 2 ? 0 : size_t(m) * k, strideB = sb.size() == 2 ? 0 : size_t(k) * n;
  std::vector<float> got = tfcc::data::get(r), gotb = tfcc::data::get(rb);
  bool ok = true;
  for (unsigned bi = 0; bi < batch && ok; ++bi)
    for (unsigned i = 0; i < m && ok; ++i)
      for (unsigned j = 0; j < n; ++j) {
        double s = 0;
        for (unsigned p = 0; p < k; ++p) s += double(ha[bi * strideA + i * k + p]) * double(hb[bi * strideB + p * n + j]);
        size_t idx = (size_t(bi) * m + i) * n + j;
        if (!is_similar(got[idx], float(s)) || !is_similar(gotb[idx], float(s + hbias[j]))) {
          ok = false;
          break;
        }
      }
  CHECK(ok);
}

static void test_blas() {
  // the four shape families of tfcc/test/python/testcase/blas/matmul.py:25-69, m, n, k in [1, 100)
  std::mt19937 rng(1234);
  std::uniform_int_distribution<unsigned> dim(1, 99), bdim(1, 5);
  for (int rep = 0; rep < 5; ++rep) {
    unsigned m = dim(rng), n = dim(rng), k = dim(rng), b1 = bdim(rng), b2 = bdim(rng);
    matmul_case(rng, {m, k}, {k, n});
    matmul_case(rng, {b1, m, k}, {k, n});
    matmul_case(rng, {m, k}, {b1, k, n});
    matmul_case(rng, {b1, b2, m, k}, {b1, b2, k, n});
  }
}

static void test_matmul_broadcast() {
  // a leading dimension of 1 on one side is broadcast (beyond tfcc/core/operations/tfcc_blas.cpp:36-42)
  std::mt19937 rng(3);
  std::uniform_real_distribution<float> dist(-1.f, 1.f);
  const unsigned batch = 3, heads = 2, m = 5, k = 8, n = 4;
  std::vector<float> ha(batch * heads * m * k), hb(heads * k * n);
  for (auto& v : ha) v = dist(rng);
  for (auto& v : hb) v = dist(rng);
  tfcc::Variable<float> a = tfcc::data::set(ha, {batch, heads, m, k});
  tfcc::Variable<float> b = tfcc::data::set(hb, {1, heads, k, n});
  tfcc::Variable<float> c = tfcc::blas::matmul(a, b);
  CHECK((c.shape() == tfcc::Shape({batch, heads, m, n})));
  std::vector<float> got = tfcc::data::get(c);
  bool ok = true;
  for (unsigned x = 0; x < batch; ++x)
    for (unsigned h = 0; h < heads; ++h)
      for (unsigned i = 0; i < m; ++i)
        for (unsigned j = 0; j < n; ++j) {
          double s = 0;
          for (unsigned p = 0; p < k; ++p) s += double(ha[((x * heads + h) * m + i) * k + p]) * double(hb[(h * k + p) * n + j]);
          ok = ok && is_similar(got[((x * heads + h) * m + i) * n + j], float(s));
        }
  CHECK(ok);
  tfcc::Variable<float> bad({2, heads, k, n});
  CHECK_THROWS_MSG(tfcc::blas::matmul(a, bad), tfcc::InvalidArgumentError, "shape invalid");
}

static void test_dequantize_requantize_known_answers() {
  // tfcc/test/quantization.cpp:62-102
  tfcc::Variable<int8_t> a = tfcc::data::set(std::vector<int8_t>{23, -115, -128, 127, -20, -11}, {6});
  tfcc::Variable<float> minV = tfcc::data::set(std::vector<float>{-2.5f}, {1}), maxV = tfcc::data::set(std::vector<float>{3.4f}, {1});
  std::vector<float> expect = {9.9372554e-01f, -2.1992157e+00f, -2.5000000e+00f, 3.4000001e+00f, -1.1765957e-03f, 2.0705891e-01f};
  std::vector<float> got = tfcc::data::get(tfcc::quantization::dequantize(a, minV, maxV));
  const float span = 3.4f - (-2.5f);
  for (size_t i = 0; i < 6; ++i) CHECK(is_similar(got[i] + span, expect[i] + span));
  tfcc::Variable<float> minO = tfcc::data::set(std::vector<float>{-12.7f}, {1}), maxO = tfcc::data::set(std::vector<float>{24.5f}, {1});
  std::vector<uint16_t> q = tfcc::data::get(tfcc::quantization::requantize<uint16_t>(a, minV, maxV, minO, maxO));
  CHECK((q == std::vector<uint16_t>{24125, 18500, 17970, 28364, 22372, 22739}));
  tfcc::Variable<float> bad({2});
  CHECK_THROWS_MSG(tfcc::quantization::dequantize(a, bad, maxV), tfcc::InvalidArgumentError, "invalid minValue");
  CHECK_THROWS_MSG(tfcc::quantization::requantize<uint16_t>(a, minV, maxV, minO, bad), tfcc::InvalidArgumentError, "invalid maxOutput");
}

static tfcc::Variable<float> quantized_matmul(const tfcc::Tensor<float>& a, const tfcc::Tensor<float>& b) {
  // tfcc/test/quantization.cpp:105-121
  tfcc::Variable<uint8_t> qa;
  tfcc::Variable<int8_t> qb;
  tfcc::Variable<float> minA, maxA, minB, maxB, minC, maxC;
  std::tie(qa, minA, maxA) = tfcc::quantization::quantize<uint8_t>(a);
  std::tie(qb, minB, maxB) = tfcc::quantization::quantize<int8_t>(b);
  tfcc::Variable<int32_t> ra = tfcc::rocm::quantization::reduce_sum(qa, true);
  tfcc::Variable<int32_t> rb = tfcc::rocm::quantization::reduce_sum(qb, false);
  tfcc::Variable<int32_t> qc;
  std::tie(qc, minC, maxC) = tfcc::rocm::quantization::matmul(qa, ra, minA, maxA, qb, rb, minB, maxB);
  return tfcc::quantization::dequantize(qc, minC, maxC);
}

static void test_quantized_matmul_round_trips() {
  // tfcc/test/quantization.cpp:123-189: batched x batched, matrix x batched, batched x matrix
  struct Case { std::vector<unsigned> sa, sb; };
  for (const Case& c : {Case{{2, 3, 2}, {2, 2, 1}}, Case{{3, 2}, {2, 2, 1}}, Case{{2, 3, 2}, {2, 1}}}) {
    std::vector<float> va, vb;
    for (unsigned i = 0; i < tfcc::Shape(c.sa).area(); ++i) va.push_back(float(i % 6 + 1));
    for (unsigned i = 0; i < tfcc::Shape(c.sb).area(); ++i) vb.push_back(float(i % 2 + 1));
    tfcc::Variable<float> v1 = tfcc::data::set(va, tfcc::Shape(c.sa)), v2 = tfcc::data::set(vb, tfcc::Shape(c.sb));
    std::vector<float> vr = tfcc::data::get(quantized_matmul(v1, v2));
    CHECK(vr.size() == 6);
    const int expect[6] = {5, 11, 17, 5, 11, 17};
    for (size_t i = 0; i < 6 && i < vr.size(); ++i) CHECK(static_cast<int>(vr[i]) == expect[i]);
  }
}

static void test_quantized_matmul_exact() {
  // tfcc/test/quantization.cpp:191-218 with the generator of
  // tfcc/test/python/testcase/quantization/mklquantizationmatmul.py:35-75 (seeded here)
  std::mt19937 rng(99);
  auto offset_of = [](float mn, float mx) {
    double range = double(mx - mn) * (256.0 / 255.0);
    return static_cast<long long>(std::round(double(mn) * (256.0 / range)));
  };
  for (int rep = 0; rep < 9; ++rep) {
    unsigned m, n, k = std::uniform_int_distribution<unsigned>(1, 511)(rng);
    if (rep % 3 == 0) { n = std::uniform_int_distribution<unsigned>(1, 127)(rng); m = n * 6 + std::uniform_int_distribution<unsigned>(1, 127)(rng); }
    else if (rep % 3 == 1) { m = std::uniform_int_distribution<unsigned>(1, 511)(rng); n = m / 6 + std::uniform_int_distribution<unsigned>(1, 127)(rng); }
    else { m = std::uniform_int_distribution<unsigned>(1, 511)(rng); n = 1; }
    std::uniform_real_distribution<float> lo(-5.f, 5.f), width(0.05f, 5.f);
    float aMin = lo(rng), aMax = aMin + width(rng), bMin = lo(rng), bMax = bMin + width(rng);
    std::vector<uint8_t> ha(size_t(m) * k);
    std::vector<int8_t> hb(size_t(k) * n);
    for (auto& v : ha) v = uint8_t(rng() & 255);
    for (auto& v : hb) v = int8_t(int(rng() % 255) - 128);
    const long long oa = offset_of(aMin, aMax), ob = offset_of(bMin, bMax) + 128;
    tfcc::Variable<uint8_t> a = tfcc::data::set(ha, {m, k});
    tfcc::Variable<int8_t> b = tfcc::data::set(hb, {k, n});
    tfcc::Variable<float> tAmin = tfcc::data::set(std::vector<float>{aMin}, {1}), tAmax = tfcc::data::set(std::vector<float>{aMax}, {1});
    tfcc::Variable<float> tBmin = tfcc::data::set(std::vector<float>{bMin}, {1}), tBmax = tfcc::data::set(std::vector<float>{bMax}, {1});
    tfcc::Variable<int32_t> ra = tfcc::rocm::quantization::reduce_sum(a, true), rb = tfcc::rocm::quantization::reduce_sum(b, false);
    tfcc::Variable<int32_t> result;
    tfcc::Variable<float> minC, maxC;
    std::tie(result, minC, maxC) = tfcc::rocm::quantization::matmul(a, ra, tAmin, tAmax, b, rb, tBmin, tBmax);
    std::vector<int32_t> got = tfcc::data::get(result);
    bool ok = got.size() == size_t(m) * n;
    for (unsigned i = 0; i < m && ok; ++i)
      for (unsigned j = 0; j < n; ++j) {
        long long s = 0;
        for (unsigned p = 0; p < k; ++p) s += (ha[size_t(i) * k + p] + oa) * (hb[size_t(p) * n + j] + ob);
        if (got[size_t(i) * n + j] != static_cast<int32_t>(static_cast<uint32_t>(s))) { ok = false; break; }
      }
    CHECK(ok);
    // fused requantize gives the same bytes as the separate pass
    float lvl = tfcc::data::get(maxC)[0] / 2147483648.0f;
    tfcc::Variable<float> minO = tfcc::data::set(std::vector<float>{-float(k) * 3000.f * lvl}, {1});
    tfcc::Variable<float> maxO = tfcc::data::set(std::vector<float>{float(k) * 3000.f * lvl}, {1});
    tfcc::Variable<uint8_t> separate = tfcc::quantization::requantize<uint8_t>(result, minC, maxC, minO, maxO);
    tfcc::Variable<uint8_t> fused;
    tfcc::Variable<int32_t> acc;
    std::tie(fused, std::ignore, std::ignore) =
        tfcc::rocm::quantization::matmul_requantize(a, ra, tAmin, tAmax, b, rb, tBmin, tBmax, minO, maxO, &acc);
    CHECK(tfcc::data::get(fused) == tfcc::data::get(separate));
    CHECK(tfcc::data::get(acc) == got);
  }
  // weights prepared once (column sums + packed copy): the same int32 result as the plain call, for decode
  // shapes (the packed copy is streamed) and for more rows than that (the weights themselves are read)
  for (unsigned m : {1u, 5u, 8u, 9u, 40u}) {
    const unsigned k = 512, n = 2064;
    std::vector<uint8_t> ha(size_t(m) * k);
    std::vector<int8_t> hb(size_t(k) * n);
    for (auto& v : ha) v = uint8_t(rng() & 255);
    for (auto& v : hb) v = int8_t(int(rng() % 255) - 128);
    tfcc::Variable<uint8_t> a = tfcc::data::set(ha, {m, k});
    tfcc::Variable<int8_t> b = tfcc::data::set(hb, {k, n});
    tfcc::Variable<float> tAmin = tfcc::data::set(std::vector<float>{-1.5f}, {1}), tAmax = tfcc::data::set(std::vector<float>{2.25f}, {1});
    tfcc::Variable<float> tBmin = tfcc::data::set(std::vector<float>{-0.75f}, {1}), tBmax = tfcc::data::set(std::vector<float>{0.5f}, {1});
    tfcc::Variable<int32_t> ra = tfcc::rocm::quantization::reduce_sum(a, true), rb = tfcc::rocm::quantization::reduce_sum(b, false);
    tfcc::rocm::quantization::PreparedWeights w(b);
    CHECK(tfcc::data::get(w.reduceSum()) == tfcc::data::get(rb));
    tfcc::Variable<int32_t> plain, prepared;
    tfcc::Variable<float> minC, maxC, minP, maxP;
    std::tie(plain, minC, maxC) = tfcc::rocm::quantization::matmul(a, ra, tAmin, tAmax, b, rb, tBmin, tBmax);
    std::tie(prepared, minP, maxP) = tfcc::rocm::quantization::matmul(a, ra, tAmin, tAmax, w, tBmin, tBmax);
    CHECK(tfcc::data::get(prepared) == tfcc::data::get(plain));
    CHECK(tfcc::data::get(minP) == tfcc::data::get(minC) && tfcc::data::get(maxP) == tfcc::data::get(maxC));
    if (m == 5) {  // and against the definition
      const long long oa = offset_of(-1.5f, 2.25f), ob = offset_of(-0.75f, 0.5f) + 128;
      std::vector<int32_t> got = tfcc::data::get(prepared);
      bool ok = true;
      for (unsigned i = 0; i < m && ok; ++i)
        for (unsigned j = 0; j < n; j += 7) {
          long long sum = 0;
          for (unsigned q = 0; q < k; ++q) sum += (ha[size_t(i) * k + q] + oa) * (hb[size_t(q) * n + j] + ob);
          if (got[size_t(i) * n + j] != static_cast<int32_t>(static_cast<uint32_t>(sum))) { ok = false; break; }
        }
      CHECK(ok);
    }
  }
  // error texts of tfcc/mkl/operations/tfcc_mklquantization.cpp:75-118
  tfcc::Variable<uint8_t> a({4, 8});
  tfcc::Variable<int8_t> b({8, 3}), bBad({7, 3});
  tfcc::Variable<int32_t> ra({4}), rb({3}), rWrong({5});
  tfcc::Variable<float> one({1}), two({2});
  CHECK_THROWS_MSG(tfcc::rocm::quantization::matmul(a, ra, one, one, bBad, rb, one, one), tfcc::InvalidArgumentError, "tensor a and b don't match");
  CHECK_THROWS_MSG(tfcc::rocm::quantization::matmul(a, rWrong, one, one, b, rb, one, one), tfcc::InvalidArgumentError, "tensor a and reduceSumA don't match");
  CHECK_THROWS_MSG(tfcc::rocm::quantization::matmul(a, ra, two, one, b, rb, one, one), tfcc::InvalidArgumentError, "invalid tensor minA");
}

static void test_layer_ops() {
  std::mt19937 rng(7);
  std::normal_distribution<float> dist(0.f, 1.f);
  std::vector<float> hx(4 * 6 * 8);
  for (auto& v : hx) v = dist(rng);
  tfcc::Variable<float> x = tfcc::data::set(hx, {4, 6, 8});
  std::vector<float> sm = tfcc::data::get(tfcc::math::softmax(x, 2));
  for (unsigned r = 0; r < 24; ++r) {
    float s = 0;
    for (unsigned c = 0; c < 8; ++c) s += sm[r * 8 + c];
    CHECK(std::fabs(s - 1.f) < 1e-5f);
  }
  CHECK_THROWS(tfcc::math::softmax(x, 3), tfcc::InvalidArgumentError);
  std::vector<float> t = tfcc::data::get(tfcc::base::transpose(x, {0, 2, 1}));
  CHECK(t[1] == hx[8] && t[6] == hx[1]);
  std::vector<float> g = tfcc::data::get(tfcc::math::gelu_accurate(x));
  CHECK(is_similar(g[0], float(0.5 * hx[0] * (1 + std::erf(hx[0] / std::sqrt(2.0))))));
  tfcc::Variable<float> bias = tfcc::data::set(std::vector<float>(8, 2.f), {8});
  std::vector<float> added = tfcc::data::get(x + bias), scaled = tfcc::data::get(x * 0.125f);
  CHECK(added[5] == hx[5] + 2.f && scaled[5] == hx[5] * 0.125f);
  tfcc::Variable<float> gamma = tfcc::data::set(std::vector<float>(8, 1.f), {8}), beta = tfcc::data::set(std::vector<float>(8, 0.f), {8});
  std::vector<float> ln = tfcc::data::get(tfcc::nn::layer_normalization(x, gamma, beta, 1e-12f, 2));
  float mean = 0;
  for (unsigned c = 0; c < 8; ++c) mean += ln[c];
  CHECK(std::fabs(mean) < 1e-5f);
}

// tfcc/test/rnn.cpp:126-175 with the generators of tfcc/test/python/testcase/rnn/lstmforward.py and
// lstmbackward.py (seeded here): sequences of 1-7 steps, batch 1-4, 32-63 units and inputs; expectations
// from the same recurrence in double.
static void test_lstm_sequences() {
  std::mt19937 rng(2024);
  std::uniform_real_distribution<float> dist(-1.f, 1.f);
  auto sig = [](double v) { return 1.0 / (1.0 + std::exp(-v)); };
  for (int round = 0; round < 6; ++round) {
    const bool backward = round % 2 == 1;
    const unsigned seq = 1 + rng() % 7, batch = 1 + rng() % 4, hidden = 32 + rng() % 32, length = 32 + rng() % 32;
    std::vector<float> ha(size_t(seq) * batch * length), wi(size_t(length) * 4 * hidden), wh(size_t(hidden) * 4 * hidden),
        hb(4 * hidden), hih(size_t(batch) * hidden), hic(size_t(batch) * hidden);
    for (auto* v : {&ha, &wi, &wh, &hb, &hih, &hic})
      for (auto& x : *v) x = dist(rng);
    std::vector<double> h(hih.begin(), hih.end()), c(hic.begin(), hic.end()), want;
    for (unsigned step = 0; step < seq; ++step) {
      const unsigned t = backward ? seq - 1 - step : step;
      std::vector<double> nh(h.size()), nc(c.size());
      for (unsigned b = 0; b < batch; ++b)
        for (unsigned u = 0; u < hidden; ++u) {
          double g[4];
          for (unsigned q = 0; q < 4; ++q) {
            double acc = hb[q * hidden + u];
            for (unsigned p = 0; p < length; ++p)
              acc += double(ha[(size_t(t) * batch + b) * length + p]) * wi[size_t(p) * 4 * hidden + q * hidden + u];
            for (unsigned p = 0; p < hidden; ++p) acc += h[size_t(b) * hidden + p] * wh[size_t(p) * 4 * hidden + q * hidden + u];
            g[q] = acc;
          }
          nc[size_t(b) * hidden + u] = std::tanh(g[1]) * sig(g[0]) + c[size_t(b) * hidden + u] * sig(g[2]);
          nh[size_t(b) * hidden + u] = std::tanh(nc[size_t(b) * hidden + u]) * sig(g[3]);
        }
      h = nh;
      c = nc;
      want.insert(want.end(), h.begin(), h.end());
    }
    tfcc::Variable<float> a = tfcc::data::set(ha, {seq, batch, length}), ik = tfcc::data::set(wi, {length, 4 * hidden}),
                          sk = tfcc::data::set(wh, {hidden, 4 * hidden}), bias = tfcc::data::set(hb, {4 * hidden}),
                          ih = tfcc::data::set(hih, {batch, hidden}), ic = tfcc::data::set(hic, {batch, hidden});
    tfcc::Variable<float> result, rh, rc;
    std::tie(result, rh, rc) = backward ? tfcc::rnn::lstm_backward(a, ik, sk, bias, ih, ic)
                                        : tfcc::rnn::lstm_forward(a, ik, sk, bias, ih, ic);
    CHECK(result.shape() == tfcc::Shape({seq, batch, hidden}) && rh.shape() == ih.shape() && rc.shape() == ic.shape());
    std::vector<float> got = tfcc::data::get(result), gh = tfcc::data::get(rh), gc = tfcc::data::get(rc);
    bool ok = got.size() == want.size();
    for (size_t i = 0; ok && i < got.size(); ++i) ok = is_similar(got[i], float(want[i]));
    for (size_t i = 0; ok && i < gh.size(); ++i) ok = is_similar(gh[i], float(h[i])) && is_similar(gc[i], float(c[i]));
    CHECK(ok);
    // the checks of tfcc/core/operations/tfcc_rnn.cpp:33-53
    tfcc::Variable<float> badBias({4 * hidden + 1}), badState({hidden + 1, 4 * hidden}), flat({seq * batch, length});
    CHECK_THROWS_MSG(tfcc::rnn::lstm_forward(flat, ik, sk, bias, ih, ic), tfcc::InvalidArgumentError, "invalid input");
    CHECK_THROWS_MSG(tfcc::rnn::lstm_forward(a, ik, sk, badBias, ih, ic), tfcc::InvalidArgumentError, "invalid bias");
    CHECK_THROWS_MSG(tfcc::rnn::lstm_backward(a, ik, badState, bias, ih, ic), tfcc::InvalidArgumentError, "invalid state kernel");
    if (length != hidden)
      CHECK_THROWS_MSG(tfcc::rnn::lstm_forward(a, sk, sk, bias, ih, ic), tfcc::InvalidArgumentError, "invalid input kernel");
    CHECK_THROWS_MSG(tfcc::rnn::lstm_forward(a, ik, sk, bias, ih, bias), tfcc::InvalidArgumentError, "invalid ih or ic");
  }
}

// The four cells of tfcc/test/rnn.cpp:36-124 at the level of CellInterface: results against the formulas of the
// interface's own documentation (tfcc/core/interfaces/tfcc_cellinterface.h:33-86) in double.
static void test_cells() {
  std::mt19937 rng(77);
  std::uniform_real_distribution<float> dist(-2.f, 2.f);
  auto sig = [](double v) { return 1.0 / (1.0 + std::exp(-v)); };
  const unsigned batch = 3, units = 70, inputSize = 19;
  auto make = [&](std::vector<unsigned> shape, std::vector<float>& host) {
    size_t n = 1;
    for (unsigned d : shape) n *= d;
    host.resize(n);
    for (auto& v : host) v = dist(rng);
    return tfcc::data::set(host, tfcc::Shape(shape));
  };
  std::vector<float> hs, hx4, hh4, hb4, hx3, hh3, hb2, hv2, hin, hcv, hcb, hbi, hbh;
  tfcc::Variable<float> state = make({batch, units}, hs), x4 = make({batch, 4 * units}, hx4), h4 = make({batch, 4 * units}, hh4),
                        b4 = make({4 * units}, hb4), x3 = make({batch, 3 * units}, hx3), h3 = make({batch, 3 * units}, hh3),
                        b2 = make({2 * units}, hb2), v2 = make({batch, 2 * units}, hv2), in = make({batch, inputSize}, hin),
                        cv = make({batch, units}, hcv), cb = make({units}, hcb), bi = make({units}, hbi), bh = make({units}, hbh);
  tfcc::CellInterface<float>& cell = tfcc::Operation<float>::getCurrentInterface().getCellInterface();
  tfcc::Variable<float> h, cs;
  std::tie(h, cs) = cell.processLSTMCell(state, x4, h4, b4, 1.0f);
  std::vector<float> gh = tfcc::data::get(h), gcs = tfcc::data::get(cs), gates = tfcc::data::get(cell.processGRUCellGates(state, in, v2, b2)),
                     cand = tfcc::data::get(cell.processGRUCellCandidate(state, v2, b2, cv, cb)),
                     pt = tfcc::data::get(cell.processPyTorchGRUCell(state, x3, h3, b2, bi, bh));
  bool ok = true;
  for (unsigned b = 0; b < batch; ++b)
    for (unsigned u = 0; u < units; ++u) {
      auto pre4 = [&](unsigned q) { return double(hx4[b * 4 * units + q * units + u]) + hh4[b * 4 * units + q * units + u] + hb4[q * units + u]; };
      const double c = std::tanh(pre4(1)) * sig(pre4(0)) + hs[b * units + u] * sig(pre4(2) + 1.0);
      ok = ok && is_similar(gcs[b * units + u], float(c)) && is_similar(gh[b * units + u], float(std::tanh(c) * sig(pre4(3))));
      const double r = sig(double(hv2[b * 2 * units + u]) + hb2[u]), z = sig(double(hv2[b * 2 * units + units + u]) + hb2[units + u]);
      ok = ok && is_similar(gates[b * (inputSize + units) + inputSize + u], float(r * hs[b * units + u]));
      ok = ok && is_similar(cand[b * units + u], float(z * hs[b * units + u] + (1 - z) * std::tanh(double(hcv[b * units + u]) + hcb[u])));
      const double pr = sig(double(hx3[b * 3 * units + u]) + hh3[b * 3 * units + u] + hb2[u]);
      const double pz = sig(double(hx3[b * 3 * units + units + u]) + hh3[b * 3 * units + units + u] + hb2[units + u]);
      const double n = std::tanh(double(hx3[b * 3 * units + 2 * units + u]) + hbi[u] + pr * (double(hh3[b * 3 * units + 2 * units + u]) + hbh[u]));
      ok = ok && is_similar(pt[b * units + u], float(n + pz * (hs[b * units + u] - n)));
    }
  for (unsigned b = 0; b < batch; ++b)
    for (unsigned j = 0; j < inputSize; ++j) ok = ok && gates[b * (inputSize + units) + j] == hin[b * inputSize + j];
  CHECK(ok);
  CHECK_THROWS_MSG(cell.processLSTMCell(state, x3, h4, b4, 0.f), tfcc::InvalidArgumentError, "invalid inputValue");
  CHECK_THROWS_MSG(cell.processLSTMCell(state, x4, h3, b4, 0.f), tfcc::InvalidArgumentError, "invalid stateHValue");
  CHECK_THROWS_MSG(cell.processLSTMCell(b4, x4, h4, b4, 0.f), tfcc::InvalidArgumentError, "invalid stateC");
  CHECK_THROWS_MSG(cell.processGRUCellGates(state, in, x4, b2), tfcc::InvalidArgumentError, "invalid value");
  CHECK_THROWS_MSG(cell.processGRUCellCandidate(state, v2, b2, cv, b2), tfcc::InvalidArgumentError, "invalid cBias");
  CHECK_THROWS_MSG(cell.processPyTorchGRUCell(state, x3, h3, b2, bi, b2), tfcc::InvalidArgumentError, "invalid candidateHBias");
}

// Scopes, the npz loader, constants and configures on any device (tfcc/test/scope.cpp, framework.cpp).
static void test_scopes_and_constants() {
  CHECK(tfcc::Scope::getCurrentScope().getFullName() == "");
  {
    auto a = tfcc::Scope::scope("layer");
    auto b = tfcc::Scope::scope("dense");
    CHECK(tfcc::Scope::getCurrentScope().getFullName() == "layer/dense/");
    CHECK(&tfcc::Scope::getRootScope().getChild("layer").getChild("dense") == &tfcc::Scope::getCurrentScope());
    {
      tfcc::ScopeGuard moved = tfcc::Scope::scope("0");
      tfcc::ScopeGuard target(std::move(moved));  // only the target pops
      CHECK(tfcc::Scope::getCurrentScope().getFullName() == "layer/dense/0/");
      CHECK(tfcc::Configure<unsigned>::getConfigure("units") > 0);
      CHECK(tfcc::Configure<unsigned>::getConfigure("absent", 5u) == 5u);
      CHECK_THROWS(tfcc::Configure<unsigned>::getConfigure("absent"), tfcc::RuntimeError);
      tfcc::Constant<float>& k = tfcc::Constant<float>::getConstant("dense/kernel");
      CHECK(k.shape().size() == 2 && k.available() && k.data() != nullptr);
      tfcc::Constant<float>& t = tfcc::Constant<float>::getConstant("dense/bias");
      std::vector<float> bias = tfcc::data::get(t);
      CHECK(bias.size() == k.shape(1));
      // an integer view of a float array converts element by element (tfcc/core/utils/tfcc_commutils.cpp:411-436)
      std::vector<int32_t> asInt = tfcc::data::get(tfcc::Constant<int32_t>::getConstant("dense/bias"));
      bool same = asInt.size() == bias.size();
      for (size_t i = 0; same && i < bias.size(); ++i) same = asInt[i] == static_cast<int32_t>(bias[i]);
      CHECK(same);
    }
    CHECK(tfcc::Scope::getCurrentScope().getFullName() == "layer/dense/");
    CHECK(tfcc::Configure<uint64_t>::getConfigure("__count__") >= 1);
  }
  CHECK(tfcc::Scope::getCurrentScope().getFullName() == "");
  CHECK(tfcc::DataLoader::getGlobalDefault()->hasData("rnn/lstmcell/0/inputs"));
  CHECK(!tfcc::DataLoader::getGlobalDefault()->hasData("rnn/lstmcell/0/nothing"));
  CHECK(tfcc::DataLoader::getGlobalDefault()->getAllNames().size() > 10);
}

// is_similar over whole tensors, as tfcc::is_similar (tfcc/core/utils/tfcc_debugutils.cpp) is used by the
// reference's tests
static bool all_similar(const tfcc::Tensor<float>& a, const tfcc::Tensor<float>& b) {
  if (a.shape() != b.shape()) return false;
  std::vector<float> x = tfcc::data::get(a), y = tfcc::data::get(b);
  for (size_t i = 0; i < x.size(); ++i)
    if (!is_similar(x[i], y[i])) return false;
  return true;
}

// Sequence lengths of the cell classes (tfcc/core/rnn/tfcc_lstmcell.cpp:81-91): at `step`, a row whose length is
// at most `step` keeps the state it came with, the others take the new one.
static std::vector<unsigned> alternating_lengths(unsigned batch, unsigned step) {
  std::vector<unsigned> lengths(batch);
  for (unsigned r = 0; r < batch; ++r) lengths[r] = r % 2 == 0 ? step : step + 1;  // even rows have ended
  return lengths;
}
static bool rows_follow_lengths(const tfcc::Tensor<float>& got, const tfcc::Tensor<float>& kept,
                                const tfcc::Tensor<float>& fresh, const std::vector<unsigned>& lengths, unsigned step) {
  if (got.shape() != kept.shape() || got.shape() != fresh.shape() || got.shape().size() != 2) return false;
  std::vector<float> g = tfcc::data::get(got), k = tfcc::data::get(kept), f = tfcc::data::get(fresh);
  const unsigned cols = got.shape(1);
  for (unsigned r = 0; r < got.shape(0); ++r)
    for (unsigned c = 0; c < cols; ++c) {
      const size_t i = static_cast<size_t>(r) * cols + c;
      if (step >= lengths[r] ? g[i] != k[i] : !is_similar(g[i], f[i])) return false;
    }
  return true;
}

// tfcc/test/rnn.cpp:81-104, data named as tfcc/test/python/createtestdata.py names it
// ("rnn/lstmcell/<i>/..."), generated by the Python side of this test with the formulas of
// tfcc/test/python/testcase/rnn/lstmcell.py:31-44.
static void test_lstmcell_from_constants() {
  auto scope1 = tfcc::Scope::scope("rnn");
  auto scope2 = tfcc::Scope::scope("lstmcell");
  size_t count = tfcc::Configure<uint64_t>::getConfigure("__count__");
  CHECK(count > 0);
  for (size_t i = 0; i < count; ++i) {
    auto scope3 = tfcc::Scope::scope(std::to_string(i));
    unsigned units = tfcc::Configure<unsigned>::getConfigure("units");
    tfcc::rnn::LSTMCell<float> cell(units);
    tfcc::Constant<float>& inputs = tfcc::Constant<float>::getConstant("inputs");
    tfcc::rnn::LSTMCell<float>::State state;
    state.h = tfcc::data::copy(tfcc::Constant<float>::getConstant("h"));
    state.cs = tfcc::data::copy(tfcc::Constant<float>::getConstant("cs"));
    tfcc::Constant<float>& expect = tfcc::Constant<float>::getConstant("expect");
    tfcc::Constant<float>& expectCs = tfcc::Constant<float>::getConstant("ecs");
    tfcc::Variable<float> result;
    tfcc::rnn::LSTMCell<float>::State nextState;
    std::tie(result, nextState) = cell(inputs, state, 0, {});
    CHECK(all_similar(result, expect));
    CHECK(all_similar(nextState.h, expect));
    CHECK(all_similar(nextState.cs, expectCs));
    CHECK_THROWS(cell(inputs, state, 0, {1u, 2u, 3u, 4u, 5u, 6u, 7u}), tfcc::InvalidArgumentError);
    {
      const std::vector<unsigned> lengths = alternating_lengths(inputs.shape(0), 3);
      std::tie(result, nextState) = cell(inputs, state, 3, lengths);
      CHECK(rows_follow_lengths(result, state.h, expect, lengths, 3));
      CHECK(rows_follow_lengths(nextState.h, state.h, expect, lengths, 3));
      CHECK(rows_follow_lengths(nextState.cs, state.cs, expectCs, lengths, 3));
      std::tie(result, nextState) = cell(inputs, state, 2, lengths);  // one step earlier every row is still running
      CHECK(all_similar(nextState.cs, expectCs));
    }
    // the same constant asked for again is the same object; under another scope it is looked up anew
    CHECK(&tfcc::Constant<float>::getConstant("inputs") == &inputs);
    auto other = tfcc::Scope::scope("nowhere");
    const std::string missing = "Name: [rnn/lstmcell/" + std::to_string(i) + "/nowhere/inputs] not found in data loader";
    CHECK_THROWS_MSG(tfcc::Constant<float>::getConstant("inputs"), tfcc::RuntimeError, missing.c_str());
  }
}

// tfcc/test/rnn.cpp:36-54 and 106-124: the two GRU cells, data as tfcc/test/python/testcase/rnn/grucell.py and
// pytorchgrucell.py make it ("rnn/grucell/<i>/...", "rnn/pytorch_grucell/<i>/...").
static void test_grucells_from_constants() {
  auto scope1 = tfcc::Scope::scope("rnn");
  {
    auto scope2 = tfcc::Scope::scope("grucell");
    size_t count = tfcc::Configure<uint64_t>::getConfigure("__count__");
    CHECK(count > 0);
    for (size_t i = 0; i < count; ++i) {
      auto scope3 = tfcc::Scope::scope(std::to_string(i));
      unsigned units = tfcc::Configure<unsigned>::getConfigure("units");
      tfcc::rnn::GRUCell<float> cell(units);
      tfcc::Constant<float>& inputs = tfcc::Constant<float>::getConstant("inputs");
      tfcc::Variable<float> state = tfcc::data::copy(tfcc::Constant<float>::getConstant("state"));
      tfcc::Variable<float> result, nextState;
      std::tie(result, nextState) = cell(inputs, state, 0, {});
      CHECK(all_similar(result, tfcc::Constant<float>::getConstant("expect")));
      CHECK(all_similar(nextState, tfcc::Constant<float>::getConstant("expect")));
      const std::vector<unsigned> lengths = alternating_lengths(inputs.shape(0), 5);
      std::tie(result, nextState) = cell(inputs, state, 5, lengths);
      CHECK(rows_follow_lengths(nextState, state, tfcc::Constant<float>::getConstant("expect"), lengths, 5));
      CHECK(rows_follow_lengths(result, state, tfcc::Constant<float>::getConstant("expect"), lengths, 5));
      CHECK_THROWS(cell(inputs, state, 0, std::vector<unsigned>(inputs.shape(0) + 1, 1u)), tfcc::InvalidArgumentError);
    }
  }
  {
    auto scope2 = tfcc::Scope::scope("pytorch_grucell");
    size_t count = tfcc::Configure<uint64_t>::getConfigure("__count__");
    CHECK(count > 0);
    for (size_t i = 0; i < count; ++i) {
      auto scope3 = tfcc::Scope::scope(std::to_string(i));
      unsigned units = tfcc::Configure<unsigned>::getConfigure("units");
      tfcc::rnn::PyTorchGRUCell<float> cell(units);
      tfcc::Constant<float>& inputs = tfcc::Constant<float>::getConstant("inputs");
      tfcc::Variable<float> state = tfcc::data::copy(tfcc::Constant<float>::getConstant("state"));
      tfcc::Variable<float> result, nextState;
      std::tie(result, nextState) = cell(inputs, state, 0, {});
      CHECK(all_similar(result, tfcc::Constant<float>::getConstant("expect")));
      std::tie(result, nextState) = cell(inputs, state, 0, {});  // the joined kernels are kept
      CHECK(all_similar(nextState, tfcc::Constant<float>::getConstant("expect")));
      const std::vector<unsigned> lengths = alternating_lengths(inputs.shape(0), 1);
      std::tie(result, nextState) = cell(inputs, state, 1, lengths);
      CHECK(rows_follow_lengths(nextState, state, tfcc::Constant<float>::getConstant("expect"), lengths, 1));
    }
  }
}

// tfcc::base::slice / concat, tfcc::nn::gather and tfcc::data::cast on other element types than float
// (tfcc/test/base.cpp's slice and concat cases in kind): bytes moved, never converted.
static void test_data_movement() {
  std::vector<int32_t> hv(4 * 6);
  for (size_t i = 0; i < hv.size(); ++i) hv[i] = static_cast<int32_t>(i * 7) - 40;
  tfcc::Variable<int32_t> v = tfcc::data::set(hv, {4, 6});
  std::vector<int32_t> s = tfcc::data::get(tfcc::base::slice(v, 1, 2, 5));
  bool ok = s.size() == 12;
  for (unsigned r = 0; ok && r < 4; ++r)
    for (unsigned c = 0; c < 3; ++c) ok = ok && s[r * 3 + c] == hv[r * 6 + 2 + c];
  CHECK(ok);
  CHECK(tfcc::base::slice(v, 0, 3, 99).shape() == tfcc::Shape({1, 6}));
  {
    // tfcc::base::assign_to (tfcc/core/operations/tfcc_base.cpp:162-181): columns 1..2 of every row replaced
    std::vector<int32_t> pv = {100, 101, 102, 103, 104, 105, 106, 107};
    tfcc::Variable<int32_t> patch = tfcc::data::set(pv, {4, 2});
    tfcc::Variable<int32_t> target = tfcc::data::copy(v);
    tfcc::base::assign_to(patch, 1, 1, target);
    std::vector<int32_t> t = tfcc::data::get(target);
    bool same = true;
    for (unsigned r = 0; r < 4; ++r)
      for (unsigned c = 0; c < 6; ++c) same = same && t[r * 6 + c] == ((c == 1 || c == 2) ? pv[r * 2 + c - 1] : hv[r * 6 + c]);
    CHECK(same);
    CHECK_THROWS(tfcc::base::assign_to(patch, 1, 5, target), tfcc::InvalidArgumentError);
    CHECK_THROWS(tfcc::base::assign_to(patch, 2, 0, target), tfcc::InvalidArgumentError);
  }
  CHECK_THROWS_MSG(tfcc::base::slice(v, 2, 0, 1), tfcc::InvalidArgumentError, "invalid axis");
  CHECK_THROWS_MSG(tfcc::base::slice(v, 1, 3, 3), tfcc::InvalidArgumentError, "start large than end");
  CHECK_THROWS_MSG(tfcc::base::slice(v, 1, 6, 7), tfcc::InvalidArgumentError, "invalid start");
  tfcc::Variable<int32_t> left = tfcc::base::slice(v, 1, 0, 2), right = tfcc::base::slice(v, 1, 2, 6);
  CHECK(tfcc::data::get(tfcc::base::concat<int32_t>({&left, &right}, 1)) == hv);
  tfcc::Variable<int32_t> top = tfcc::base::slice(v, 0, 0, 1), rest = tfcc::base::slice(v, 0, 1, 4);
  CHECK(tfcc::data::get(tfcc::base::concat<int32_t>({&top, &rest}, 0)) == hv);
  CHECK_THROWS_MSG(tfcc::base::concat<int32_t>({&left, &top}, 1), tfcc::InvalidArgumentError, "invalid shape");
  tfcc::Variable<int64_t> idx = tfcc::data::set(std::vector<int64_t>{3, -1, 0, 4}, {2, 2});
  std::vector<int32_t> g = tfcc::data::get(tfcc::nn::gather(v, idx));
  ok = g.size() == 24;
  for (unsigned c = 0; ok && c < 6; ++c) ok = g[c] == hv[18 + c] && g[6 + c] == 0 && g[12 + c] == hv[c] && g[18 + c] == 0;
  CHECK(ok);
  std::vector<float> f = tfcc::data::get(tfcc::data::cast<float>(v));
  ok = true;
  for (size_t i = 0; i < hv.size(); ++i) ok = ok && f[i] == static_cast<float>(hv[i]);
  CHECK(ok);
  tfcc::Variable<float> fv = tfcc::data::set(std::vector<float>{-2.5f, 0.f, 3.9f, 100.25f}, {4});
  CHECK(tfcc::data::get(tfcc::data::cast<int8_t>(fv)) == (std::vector<int8_t>{-2, 0, 3, 100}));
  CHECK(tfcc::data::get(tfcc::data::cast<uint64_t>(tfcc::data::cast<double>(fv)))[3] == 100u);
  // The interface itself, as the reference declares it (tfcc/core/interfaces/tfcc_datainterface.h:40-53): one cast
  // virtual per source type, and cast_to_boolean.  Every source type into float and back out of float.
  auto& toFloat = tfcc::Operation<float>::getCurrentInterface().getDataInterface();
#define CAST_ROUND_TRIP(T, ...)                                                                       \
  {                                                                                                   \
    const std::vector<T> h{__VA_ARGS__};                                                               \
    tfcc::Variable<T> src = tfcc::data::set(h, {static_cast<unsigned>(h.size())});                     \
    std::vector<float> asFloat = tfcc::data::get(toFloat.cast(src));                                   \
    bool same = asFloat.size() == h.size();                                                           \
    for (size_t i = 0; same && i < h.size(); ++i) same = asFloat[i] == static_cast<float>(h[i]);       \
    CHECK(same);                                                                                      \
    tfcc::Variable<float> f32 = tfcc::data::set(asFloat, {static_cast<unsigned>(h.size())});           \
    CHECK(tfcc::data::get(tfcc::Operation<T>::getCurrentInterface().getDataInterface().cast(f32)) == h); \
  }
  CAST_ROUND_TRIP(float, -1.5f, 0.f, 7.25f)
  CAST_ROUND_TRIP(double, -1.5, 0.0, 7.25)
  CAST_ROUND_TRIP(int8_t, -128, 0, 127)
  CAST_ROUND_TRIP(uint8_t, 0, 1, 255)
  CAST_ROUND_TRIP(int16_t, -32768, 0, 32767)
  CAST_ROUND_TRIP(uint16_t, 0, 1, 65535)
  CAST_ROUND_TRIP(int32_t, -16777216, 0, 16777216)
  CAST_ROUND_TRIP(uint32_t, 0u, 1u, 16777216u)
  CAST_ROUND_TRIP(int64_t, -16777216, 0, 16777216)
  CAST_ROUND_TRIP(uint64_t, 0u, 1u, 16777216u)
#undef CAST_ROUND_TRIP
  tfcc::Variable<float> mixed = tfcc::data::set(std::vector<float>{0.f, -0.f, 1e-30f, -3.f, 0.f, 2.f}, {2, 3});
  tfcc::Variable<uint8_t> flags = tfcc::data::cast_to_boolean(mixed);
  CHECK(flags.shape() == mixed.shape());
  CHECK(tfcc::data::get(flags) == (std::vector<uint8_t>{0, 0, 1, 1, 0, 1}));
  tfcc::Variable<int64_t> wide = tfcc::data::set(std::vector<int64_t>{0, 1ll << 40, -1, 0}, {4});
  CHECK(tfcc::data::get(tfcc::data::cast_to_boolean(wide)) == (std::vector<uint8_t>{0, 1, 1, 0}));
}

// tfcc::layer::Dense (tfcc/core/layers/tfcc_denselayer.cpp:47-87) in the style of the reference's layer tests:
// inputs of rank 2 and 3, with and without bias, custom constant names, and its checks.
static void test_dense_from_constants() {
  auto scope1 = tfcc::Scope::scope("layer");
  auto scope2 = tfcc::Scope::scope("dense");
  size_t count = tfcc::Configure<uint64_t>::getConfigure("__count__");
  CHECK(count > 0);
  for (size_t i = 0; i < count; ++i) {
    auto scope3 = tfcc::Scope::scope(std::to_string(i));
    unsigned units = tfcc::Configure<unsigned>::getConfigure("units");
    tfcc::Constant<float>& inputs = tfcc::Constant<float>::getConstant("inputs");
    CHECK(all_similar(tfcc::layer::dense(inputs, units, true), tfcc::Constant<float>::getConstant("expect")));
    CHECK(all_similar(tfcc::layer::dense(inputs, 0u, false), tfcc::Constant<float>::getConstant("expect_nobias")));
    CHECK(all_similar(tfcc::layer::dense(inputs, units, true, "other", "w", "b"), tfcc::Constant<float>::getConstant("expect_other")));
    // with a bias the layer is one launch; it returns what matmul followed by the broadcast add returns
    tfcc::layer::Dense<float> layer(units, true);
    tfcc::Variable<float> fused = layer(inputs);
    auto inner = tfcc::Scope::scope("dense");
    tfcc::Variable<float> separate = tfcc::blas::matmul(inputs, tfcc::Constant<float>::getConstant("kernel")) +
                                     tfcc::Constant<float>::getConstant("bias");
    CHECK(tfcc::data::get(fused) == tfcc::data::get(separate));
  }
  auto scope3 = tfcc::Scope::scope("0");
  tfcc::Constant<float>& inputs = tfcc::Constant<float>::getConstant("inputs");
  CHECK_THROWS_MSG(tfcc::layer::dense(inputs, 7777u, true), tfcc::InvalidDataError, "kernel and units don't match");
  CHECK_THROWS_MSG(tfcc::layer::dense(inputs, 0u, true, "dense", "bias", "bias"), tfcc::InvalidDataError, "invalid kernel");
  CHECK_THROWS_MSG(tfcc::layer::dense(inputs, 0u, true, "dense", "kernel", "kernel"), tfcc::InvalidDataError, "invalid bias");
  tfcc::Variable<float> flat({inputs.size()}), wrong({3, inputs.shape(inputs.shape().size() - 1) + 1});
  CHECK_THROWS_MSG(tfcc::layer::dense(flat, 0u, true), tfcc::InvalidArgumentError, "invalid inputs");
  CHECK_THROWS_MSG(tfcc::layer::dense(wrong, 0u, true), tfcc::InvalidArgumentError, "inputs and kernel don't match");
}

// tfcc::math::reduce_sum / mean / prod / max / min, min / max / pow of tensors and values, clip, leaky_relu
// (tfcc/test/math.cpp's reduce and min / max cases): results against the same expressions in double on the host.
static void test_reduce_minmax_pow() {
  std::mt19937 rng(23);
  std::uniform_real_distribution<float> dist(0.6f, 1.4f);
  const unsigned d0 = 3, d1 = 5, d2 = 37;
  std::vector<float> ha(d0 * d1 * d2), hb(d2);
  for (size_t i = 0; i < ha.size(); ++i) ha[i] = (i % 3 == 1 ? -1.f : 1.f) * dist(rng);
  for (auto& v : hb) v = dist(rng);
  tfcc::Variable<float> a = tfcc::data::set(ha, {d0, d1, d2}), b = tfcc::data::set(hb, {d2});
  for (size_t keep : {size_t(1), size_t(2)}) {
    const size_t rows = keep == 1 ? d0 : d0 * d1, cols = ha.size() / rows;
    tfcc::Variable<float> sum = tfcc::math::reduce_sum(a, keep), mean = tfcc::math::reduce_mean(a, keep),
                          prod = tfcc::math::reduce_prod(a, keep), hi = tfcc::math::reduce_max(a, keep),
                          lo = tfcc::math::reduce_min(a, keep);
    CHECK(sum.shape() == (keep == 1 ? tfcc::Shape({d0, 1, 1}) : tfcc::Shape({d0, d1, 1})));
    std::vector<float> gs = tfcc::data::get(sum), gm = tfcc::data::get(mean), gp = tfcc::data::get(prod),
                       gh = tfcc::data::get(hi), gl = tfcc::data::get(lo);
    bool ok = gs.size() == rows;
    for (size_t r = 0; ok && r < rows; ++r) {
      double s = 0, p = 1;
      float mx = ha[r * cols], mn = ha[r * cols];
      for (size_t c = 0; c < cols; ++c) {
        const float v = ha[r * cols + c];
        s += v;
        p *= v;
        mx = std::max(mx, v);
        mn = std::min(mn, v);
      }
      ok = std::fabs(gs[r] - s) < 1e-4 && std::fabs(gm[r] - s / cols) < 1e-5 &&
           std::fabs(gp[r] - p) <= 1e-4 * std::fabs(p) && gh[r] == mx && gl[r] == mn;
    }
    CHECK(ok);
  }
  CHECK_THROWS_MSG(tfcc::math::reduce_sum(a, 3), tfcc::InvalidArgumentError, "invalid keep dims");
  std::vector<float> gmin = tfcc::data::get(tfcc::math::min(a, b)), gmax = tfcc::data::get(tfcc::math::max(b, a)),
                     gminv = tfcc::data::get(tfcc::math::min(a, 0.25f)), gmaxv = tfcc::data::get(tfcc::math::max(0.25f, a)),
                     gclip = tfcc::data::get(tfcc::math::clip(a, -0.75f, 1.f)),
                     gleak = tfcc::data::get(tfcc::math::leaky_relu(a, 0.1f));
  tfcc::Variable<float> mag = tfcc::math::abs(a);
  std::vector<float> gpow = tfcc::data::get(tfcc::math::pow(mag, b)), gpowv = tfcc::data::get(tfcc::math::pow(mag, 2.5f)),
                     gvpow = tfcc::data::get(tfcc::math::pow(1.5f, a));
  bool ok = gmin.size() == ha.size() && gpow.size() == ha.size() && gvpow.size() == ha.size();
  for (size_t i = 0; ok && i < ha.size(); ++i) {
    const float x = ha[i], y = hb[i % d2];
    ok = gmin[i] == std::min(x, y) && gmax[i] == std::max(x, y) && gminv[i] == std::min(x, 0.25f) &&
         gmaxv[i] == std::max(x, 0.25f) && gclip[i] == std::min(std::max(x, -0.75f), 1.f) &&
         gleak[i] == (x > 0.f ? x : x * 0.1f) &&
         std::fabs(gpow[i] - std::pow(std::fabs((double)x), (double)y)) < 2e-6 * std::pow(std::fabs((double)x), (double)y) + 1e-7 &&
         std::fabs(gpowv[i] - std::pow(std::fabs((double)x), 2.5)) < 2e-6 * std::pow(std::fabs((double)x), 2.5) + 1e-7 &&
         std::fabs(gvpow[i] - std::pow(1.5, (double)x)) < 2e-6 * std::pow(1.5, (double)x) + 1e-7;
  }
  CHECK(ok);
}

// tfcc::relation (tensor against value, value against tensor, tensor against tensor), tfcc::nn::where,
// tfcc::base::tril / triu, tfcc::math::argmax and data::fill, on float and int64 tensors
// (tfcc/test/relation.cpp, tfcc/test/nn.cpp's where cases in the reference).
static void test_relation_where_triangle() {
  std::vector<int64_t> hv(3 * 5), hw(5);
  for (size_t i = 0; i < hv.size(); ++i) hv[i] = static_cast<int64_t>((i * 7) % 5) - 2;
  for (size_t i = 0; i < hw.size(); ++i) hw[i] = static_cast<int64_t>(i) - 2;
  tfcc::Variable<int64_t> v = tfcc::data::set(hv, {3, 5}), w = tfcc::data::set(hw, {5});
  std::vector<uint8_t> eq = tfcc::data::get(tfcc::relation::equal(v, int64_t(1))),
                       lt = tfcc::data::get(tfcc::relation::less(int64_t(0), v)),   // 0 < v
                       ge = tfcc::data::get(tfcc::relation::greater_equal(v, w)),
                       ne = tfcc::data::get(tfcc::relation::unequal(w, v));
  bool ok = eq.size() == hv.size() && ge.size() == hv.size() && ne.size() == hv.size();
  for (size_t i = 0; ok && i < hv.size(); ++i)
    ok = eq[i] == (hv[i] == 1) && lt[i] == (0 < hv[i]) && ge[i] == (hv[i] - hw[i % 5] >= 0) && ne[i] == (hw[i % 5] != hv[i]);
  CHECK(ok);
  CHECK_THROWS(tfcc::relation::equal(v, tfcc::data::set(std::vector<int64_t>{1, 2}, {2})), tfcc::InvalidArgumentError);

  std::vector<float> hx(4 * 6), hy(4 * 6);
  for (size_t i = 0; i < hx.size(); ++i) {
    hx[i] = static_cast<float>((i * 5) % 7) - 3.f;
    hy[i] = static_cast<float>(i) * 0.5f;
  }
  tfcc::Variable<float> x = tfcc::data::set(hx, {4, 6}), y = tfcc::data::set(hy, {4, 6});
  tfcc::Variable<uint8_t> positive = tfcc::relation::greater(x, 0.f);
  std::vector<float> w1 = tfcc::data::get(tfcc::nn::where(positive, x, y)), w2 = tfcc::data::get(tfcc::nn::where(positive, 7.f, y)),
                     w3 = tfcc::data::get(tfcc::nn::where(positive, x, -1.f)), lo = tfcc::data::get(tfcc::base::tril(x, 1)),
                     up = tfcc::data::get(tfcc::base::triu(x, -1));
  std::vector<int64_t> am = tfcc::data::get(tfcc::math::argmax(x, 1));
  ok = w1.size() == hx.size() && am.size() == 4;
  for (size_t i = 0; ok && i < hx.size(); ++i) {
    const long r = static_cast<long>(i / 6), c = static_cast<long>(i % 6);
    ok = w1[i] == (hx[i] > 0 ? hx[i] : hy[i]) && w2[i] == (hx[i] > 0 ? 7.f : hy[i]) && w3[i] == (hx[i] > 0 ? hx[i] : -1.f) &&
         lo[i] == (c <= r + 1 ? hx[i] : 0.f) && up[i] == (c >= r - 1 ? hx[i] : 0.f);
  }
  for (size_t r = 0; ok && r < 4; ++r) {
    size_t best = 0;
    for (size_t c = 1; c < 6; ++c)
      if (hx[r * 6 + c] > hx[r * 6 + best]) best = c;
    ok = am[r] == static_cast<int64_t>(best);
  }
  CHECK(ok);
  CHECK(tfcc::math::argmax(x, 0).shape() == tfcc::Shape({1, 6}));
  CHECK_THROWS_MSG(tfcc::nn::where(positive, x, tfcc::data::set(std::vector<float>{1.f}, {1})), tfcc::InvalidArgumentError,
                   "condition x and y has different shape");
  CHECK_THROWS_MSG(tfcc::base::tril(tfcc::data::set(std::vector<float>{1.f, 2.f}, {2}), 0), tfcc::InvalidArgumentError, "invalid shape");
  tfcc::Variable<int16_t> filled(tfcc::Shape({7}));
  tfcc::data::fill(filled, static_cast<int16_t>(-3));
  CHECK(tfcc::data::get(filled) == std::vector<int16_t>(7, -3));
}

// tfcc::math::add / sub / mul / div with the broadcasting of tfcc/core/operations/tfcc_math.cpp:38-104
// (tfcc/test/math.cpp's broadcast cases): attention mask, both sides broadcast, either operand the larger.
static void test_broadcast_arithmetic() {
  std::mt19937 rng(21);
  std::uniform_real_distribution<float> dist(0.5f, 2.f);
  struct Case { std::vector<unsigned> sa, sb; };
  for (const Case& c : {Case{{2, 4, 8, 8}, {2, 1, 1, 8}}, Case{{3, 1, 5}, {1, 4, 1}}, Case{{33}, {7, 33}}, Case{{5, 6}, {1}},
                        Case{{2, 3, 4, 5, 6, 7}, {2, 1, 4, 1, 6, 1}}}) {
    size_t na = 1, nb = 1;
    for (unsigned d : c.sa) na *= d;
    for (unsigned d : c.sb) nb *= d;
    std::vector<float> ha(na), hb(nb);
    for (auto& v : ha) v = dist(rng);
    for (auto& v : hb) v = dist(rng);
    tfcc::Variable<float> a = tfcc::data::set(ha, tfcc::Shape(c.sa)), b = tfcc::data::set(hb, tfcc::Shape(c.sb));
    const size_t rank = std::max(c.sa.size(), c.sb.size());
    std::vector<unsigned> da(rank, 1), db(rank, 1), dr(rank);
    std::copy(c.sa.begin(), c.sa.end(), da.begin() + (rank - c.sa.size()));
    std::copy(c.sb.begin(), c.sb.end(), db.begin() + (rank - c.sb.size()));
    size_t total = 1;
    for (size_t d = 0; d < rank; ++d) total *= dr[d] = std::max(da[d], db[d]);
    tfcc::Variable<float> sum = a + b, dif = a - b, pro = a * b, quo = a / b;
    CHECK(sum.shape() == tfcc::Shape(dr) && quo.shape() == tfcc::Shape(dr));
    std::vector<float> gs = tfcc::data::get(sum), gd = tfcc::data::get(dif), gp = tfcc::data::get(pro), gq = tfcc::data::get(quo);
    bool ok = gs.size() == total;
    for (size_t i = 0; ok && i < total; ++i) {
      size_t rem = i, ia = 0, ib = 0, sa = 1, sb = 1;
      for (size_t d = rank; d-- > 0;) {
        const size_t coord = rem % dr[d];
        rem /= dr[d];
        ia += (da[d] == 1 ? 0 : coord) * sa;
        ib += (db[d] == 1 ? 0 : coord) * sb;
        sa *= da[d];
        sb *= db[d];
      }
      ok = gs[i] == ha[ia] + hb[ib] && gd[i] == ha[ia] - hb[ib] && gp[i] == ha[ia] * hb[ib] && gq[i] == ha[ia] / hb[ib];
    }
    CHECK(ok);
  }
  tfcc::Variable<float> a({2, 3}), b({2, 2}), e({0, 3}), one({1, 3});
  CHECK_THROWS_MSG(a + b, tfcc::InvalidArgumentError, "broadcast failed");
  CHECK((e + one).shape() == tfcc::Shape({0, 3}));
}

// Two threads, each with a session (= stream) of its own on the shared device, running the same mix of
// operations at the same time: fp32 matmul, quantize with its min/max reduction, quantized matmul.  Every
// result is checked on the thread that produced it (tfcc/core/framework/tfcc_session.h:29,60-62: device
// and session are per-thread defaults).
static void thread_body(unsigned seed, int rounds, int* failures) {
  try {
    tfcc::initialize_rocm();
    std::mt19937 rng(seed);
    std::uniform_real_distribution<float> dist(-3.f, 3.f);
    for (int round = 0; round < rounds; ++round) {
      const unsigned m = 17 + (rng() % 90), k = 8 + (rng() % 200), n = 5 + (rng() % 120);
      std::vector<float> ha(size_t(m) * k), hb(size_t(k) * n);
      for (auto& v : ha) v = dist(rng);
      for (auto& v : hb) v = dist(rng);
      tfcc::Variable<float> a = tfcc::data::set(ha, {m, k}), b = tfcc::data::set(hb, {k, n});
      std::vector<float> got = tfcc::data::get(tfcc::blas::matmul(a, b));
      for (unsigned i = 0; i < m; i += 7)
        for (unsigned j = 0; j < n; j += 5) {
          double s = 0;
          for (unsigned p = 0; p < k; ++p) s += double(ha[size_t(i) * k + p]) * double(hb[size_t(p) * n + j]);
          if (!is_similar(got[size_t(i) * n + j], float(s))) ++*failures;
        }
      // quantize finds this tensor's own range even while the other thread reduces another tensor
      tfcc::Variable<uint8_t> qa;
      tfcc::Variable<float> mn, mx;
      std::tie(qa, mn, mx) = tfcc::quantization::quantize<uint8_t>(a);
      float wantMin = ha[0], wantMax = ha[0];
      for (float v : ha) { wantMin = std::min(wantMin, v); wantMax = std::max(wantMax, v); }
      if (tfcc::data::get(mn)[0] != wantMin || tfcc::data::get(mx)[0] != wantMax) ++*failures;
      tfcc::Variable<int8_t> qb;
      tfcc::Variable<float> mnB, mxB, mnC, mxC;
      std::tie(qb, mnB, mxB) = tfcc::quantization::quantize<int8_t>(b);
      tfcc::Variable<int32_t> ra = tfcc::rocm::quantization::reduce_sum(qa, true), rb = tfcc::rocm::quantization::reduce_sum(qb, false);
      tfcc::Variable<int32_t> qc;
      std::tie(qc, mnC, mxC) = tfcc::rocm::quantization::matmul(qa, ra, mn, mx, qb, rb, mnB, mxB);
      std::vector<float> approx = tfcc::data::get(tfcc::quantization::dequantize(qc, mnC, mxC));
      // 8-bit operands: a loose bound is enough to catch results that belong to the other thread
      double err = 0, ref = 0;
      for (unsigned i = 0; i < m; i += 7)
        for (unsigned j = 0; j < n; j += 5) {
          err += std::fabs(approx[size_t(i) * n + j] - got[size_t(i) * n + j]);
          ref += std::fabs(got[size_t(i) * n + j]);
        }
      if (!(err <= 0.1 * ref + 1.0)) ++*failures;
    }
  } catch (const std::exception& e) {
    std::printf("  thread exception: %s\n", e.what());
    ++*failures;
  }
}

static void test_attention_permuted() {
  // softmax(q k^T / c) v on [batch, seq, heads, size] tensors in one launch against the operations one
  // at a time (tfcc_runtime runs Transpose, Matmul, Div, Softmax, Matmul, Transpose): the same bits
  std::mt19937 rng(5);
  std::normal_distribution<float> dist(0.f, 1.f);
  const std::vector<size_t> toHeads = {0, 2, 1, 3}, toHeadsT = {0, 2, 3, 1};
  for (auto dims : {std::array<unsigned, 5>{2, 20, 3, 8, 24}, std::array<unsigned, 5>{1, 70, 2, 64, 128}, std::array<unsigned, 5>{2, 5, 2, 12, 7}}) {
    const unsigned batch = dims[0], seq = dims[1], heads = dims[2], size = dims[3], keys = dims[4];
    std::vector<float> hq(size_t(batch) * seq * heads * size), hk(size_t(batch) * keys * heads * size), hv(hk.size());
    for (auto& x : hq) x = dist(rng);
    for (auto& x : hk) x = dist(rng);
    for (auto& x : hv) x = dist(rng);
    tfcc::Variable<float> q = tfcc::data::set(hq, {batch, seq, heads, size});
    tfcc::Variable<float> k = tfcc::data::set(hk, {batch, keys, heads, size});
    tfcc::Variable<float> v = tfcc::data::set(hv, {batch, keys, heads, size});
    const float divisor = 3.0f;
    tfcc::Variable<float> scores = tfcc::blas::matmul(tfcc::base::transpose(q, toHeads), tfcc::base::transpose(k, toHeadsT));
    tfcc::Variable<float> scaled = scores / divisor;
    tfcc::Variable<float> context = tfcc::blas::matmul(tfcc::math::softmax(scaled, 3), tfcc::base::transpose(v, toHeads));
    std::vector<float> want = tfcc::data::get(tfcc::base::transpose(context, toHeads));
    tfcc::Variable<float> fused = tfcc::rocm::blas::attention_permuted(q, toHeads, k, toHeadsT, v, toHeads, toHeads, &divisor);
    CHECK((fused.shape() == tfcc::Shape({batch, seq, heads, size})));
    CHECK(tfcc::data::get(fused) == want);
  }
  // more keys than the kernel holds in LDS: the caller is told to run the steps separately
  tfcc::Variable<float> q({1, 4, 1, 8}), k({1, 200, 1, 8}), v({1, 200, 1, 8});
  CHECK_THROWS(tfcc::rocm::blas::attention_permuted(q, toHeads, k, toHeadsT, v, toHeads, toHeads, nullptr), tfcc::NotImplementedError);
}

static void test_two_sessions_on_two_threads() {
  int f1 = 0, f2 = 0;
  std::thread t1(thread_body, 11u, 12, &f1), t2(thread_body, 23u, 12, &f2);
  t1.join();
  t2.join();
  CHECK(f1 == 0);
  CHECK(f2 == 0);
}

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "cpu";
  std::unique_ptr<tfcc::HostDevice> hostDevice;
  std::unique_ptr<tfcc::HostSession> hostSession;
  if (mode == "gpu") {
    tfcc::initialize_rocm();
  } else {
    hostDevice.reset(new tfcc::HostDevice());
    hostSession.reset(new tfcc::HostSession(*hostDevice));
    tfcc::Device::setThreadDefault(hostDevice.get());
    tfcc::Session::setThreadDefault(hostSession.get());
  }
  run("framework.reshape", test_reshape);
  run("framework.expand_dims", test_expand_dims);
  run("framework.squeeze", test_squeeze);
  run("framework.view_window", test_view_window);
  run("framework.flexallocator", test_flexallocator);
  run("framework.getdevicetype", [&] { test_device_identity(mode == "gpu" ? tfcc::DeviceType::ROCM : tfcc::DeviceType::HOST); });
  if (mode == "gpu") {
    run("blas.matmul_validation", test_matmul_validation);
    run("data.set_get_copy", test_data);
    run("blas.matmul", test_blas);
    run("blas.matmul_broadcast", test_matmul_broadcast);
    run("quantization.known_answers", test_dequantize_requantize_known_answers);
    run("quantization.rocm_matmul_round_trips", test_quantized_matmul_round_trips);
    run("quantization.rocm_matmul_exact", test_quantized_matmul_exact);
    run("layer.elementwise", test_layer_ops);
    run("math.broadcast_arithmetic", test_broadcast_arithmetic);
    run("math.reduce_minmax_pow", test_reduce_minmax_pow);
    run("relation.where_triangle", test_relation_where_triangle);
    run("layer.attention_permuted", test_attention_permuted);
    run("base.data_movement", test_data_movement);
    run("rnn.cells", test_cells);
    run("rnn.lstm_forward_backward", test_lstm_sequences);
    if (argc > 2) {  // an .npz of named test data, written by the Python side
      tfcc::NPZDataLoader loader{std::string(argv[2])};
      tfcc::DataLoader::setGlobalDefault(&loader);
      run("framework.scopes_and_constants", test_scopes_and_constants);
      run("rnn.lstmcell", test_lstmcell_from_constants);
      run("layer.dense", test_dense_from_constants);
      run("rnn.grucells", test_grucells_from_constants);
      tfcc::DataLoader::setGlobalDefault(nullptr);
    }
    run("threads.two_sessions", test_two_sessions_on_two_threads);
  } else {
    run("blas.matmul_validation", [] {
      // on the host device only the checks run; a valid shape reaches the (absent) backend
      test_matmul_validation();
      tfcc::Variable<float> a({3, 4}), b({4, 5});
      CHECK_THROWS(tfcc::blas::matmul(a, b), tfcc::NotImplementedError);
    });
    if (argc > 2) {
      tfcc::NPZDataLoader loader{std::string(argv[2])};
      tfcc::DataLoader::setGlobalDefault(&loader);
      run("framework.scopes_and_constants", test_scopes_and_constants);
      tfcc::DataLoader::setGlobalDefault(nullptr);
    }
  }
  if (mode != "gpu") {
    tfcc::Session::setThreadDefault(nullptr);
    tfcc::Device::setThreadDefault(nullptr);
  }
  std::printf("%d checks, %d failures\n", g_checks, g_failures);
  return g_failures == 0 ? 0 : 1;
}
