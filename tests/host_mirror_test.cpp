// Drives the C ABI through the C++ host mirror the way the reference's XCTest cases drive the
// Swift API: the known-answer tests of Tests/SwiftRTCoreTests/test_AlgebraicField.swift:551-597
// (matmul, its gradients via transposes, batched matmul), column-major order, a fused Dense
// forward, and the NotSupported / invalid-argument paths.  Exit code 0 = all passed.
#include <cmath>
#include <cstdio>
#include <vector>

#include "../swiftrt_amd/host/srt_host.hpp"

using namespace srt_host;

static int failures = 0;
#define EXPECT(cond) do { if (!(cond)) { std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond); ++failures; } } while (0)

static std::vector<float> arange(size_t n) { std::vector<float> v(n); for (size_t i = 0; i < n; ++i) v[i] = (float)i; return v; }

int main() {
  int count = 0;
  if (srtGetDeviceCount(&count) != srtSuccess || count < 1) { std::printf("no GPU visible\n"); return 2; }
  HipQueue q(0);

  // test_matmul
  Tensor<float> a({3, 2}, arange(6)), b({2, 4}, arange(8));
  auto c = matmul(q, a, false, b, false);
  EXPECT((c.values() == std::vector<float>{4, 5, 6, 7, 12, 17, 22, 27, 20, 29, 38, 47}));
  // its pullback for ones: dA = 1 . b^T, dB = a^T . 1
  Tensor<float> ones({3, 4}, std::vector<float>(12, 1.0f));
  EXPECT((matmul(q, ones, false, b, true).values() == std::vector<float>{6, 22, 6, 22, 6, 22}));
  EXPECT((matmul(q, a, true, ones, false).values() == std::vector<float>{6, 6, 6, 6, 9, 9, 9, 9}));
  // .t views give the same result as the flags
  EXPECT((matmul(q, a.t(), true, b.t(), true).values() == c.values()));

  // test_batchMatmul
  Tensor<float> a3({2, 3, 2}, arange(12)), b3({2, 2, 4}, arange(16));
  EXPECT((matmul(q, a3, false, b3, false).values() ==
          std::vector<float>{4, 5, 6, 7, 12, 17, 22, 27, 20, 29, 38, 47, 132, 145, 158, 171, 172, 189, 206, 223, 212, 233, 254, 275}));

  // column-major operands: the result follows lhs.order and the logical values are the same
  Tensor<float> ac({3, 2}, arange(6), Order::col), bc({2, 4}, arange(8), Order::col);
  auto cc = matmul(q, ac, false, bc, false);
  EXPECT(cc.order() == Order::col && cc.strides()[0] == 1 && cc.strides()[1] == 3);
  EXPECT(cc.values() == c.values());

  // Dense forward, fused bias + relu
  Dense<float> layer{Tensor<float>({2, 2}, {1, -1, 2, -2}), Tensor<float>({2}, {0.5f, 0.5f}), ActivationType::relu};
  Tensor<float> x({2, 2}, {1, 1, -1, -1});
  EXPECT((layer(q, x).values() == std::vector<float>{3.5f, 0.0f, 0.0f, 3.5f}));

  // its pullback: y = relu(x W + b) = [[3.5, 0], [0, 3.5]], upstream gradient [[1, 2], [3, 4]]
  //   dz = grad where y > 0 = [[1, 0], [0, 4]]; dbias = [1, 4]; dx = dz W^T; dW = x^T dz
  auto y = layer(q, x);
  auto grads = dense_backward(q, layer, x, y, Tensor<float>({2, 2}, {1, 2, 3, 4}));
  EXPECT((grads.dbias.values() == std::vector<float>{1, 4}));
  EXPECT((grads.dx.values() == std::vector<float>{1, 2, -4, -8}));
  EXPECT((grads.dweight.values() == std::vector<float>{1, -4, 1, -4}));

  // element-wise neighbours: add, mul, tensor + element, relu, and the closed forms of sigmoid / tanh at 0
  Tensor<float> p({2, 3}, {1, -2, 3, -4, 5, -6}), r({2, 3}, {0.5f, 0.5f, 0.5f, 2, 2, 2});
  EXPECT((add(q, p, r).values() == std::vector<float>{1.5f, -1.5f, 3.5f, -2, 7, -4}));
  EXPECT((mul(q, p, r).values() == std::vector<float>{0.5f, -1, 1.5f, -8, 10, -12}));
  EXPECT((add(q, p, 1.0f).values() == std::vector<float>{2, -1, 4, -3, 6, -5}));
  EXPECT((relu(q, p).values() == std::vector<float>{1, 0, 3, 0, 5, 0}));
  Tensor<float> zeros({1, 4}, std::vector<float>(4, 0.0f));
  EXPECT((sigmoid(q, zeros).values() == std::vector<float>(4, 0.5f)));
  EXPECT((tanh(q, zeros).values() == std::vector<float>(4, 0.0f)));
  EXPECT((add(q, p.t(), r.t()).values() == std::vector<float>{1.5f, -2, -1.5f, 7, 3.5f, -4}));

  // error behaviour: shape mismatch is caught before the call; double precision is NotSupported
  bool threw = false;
  try { matmul(q, a, false, a, false); } catch (const std::invalid_argument&) { threw = true; }
  EXPECT(threw);
  size_t sh[2] = {2, 2}, st[2] = {2, 1};
  srtTensorDescriptor d{srtReal64F, 2, srtOrderRow, 4, 4, sh, st, st};
  auto mem = q.allocate(64);
  EXPECT(srtMatmul(mem->pointer(), &d, 0, mem->pointer(), &d, 0, mem->pointer(), &d, q.stream()) == srtErrorNotSupported);
  try { check(srtErrorNotSupported, "x"); EXPECT(false); } catch (const NotSupported&) {}

  q.wait_for_completion();
  std::printf(failures ? "%d check(s) failed\n" : "host mirror: all checks passed\n", failures);
  return failures ? 1 : 0;
}
