// GPU test of the sycldnn:: drop-in API through backend::HIPBackend, written
// in the shape of the reference's fixtures (test/conv2d/convolution_fixture.h:
// 45-154, test/depthwise_conv2d/depthwise_conv2d_fixture.h:43-89,
// test/pooling/pooling_fixture.h:53-216): operands 1,2,3,...,max_val repeated,
// launch through the public template, wait on the returned event, compare
// with the CPU oracle (which the golden tests pin to the reference's vectors).
#include <portdnn/backend/hip_backend.h>
#include <portdnn/binaryop/launch.h>
#include <portdnn/compat/convolution.hpp>
#include <portdnn/conv2d/launch.h>
#include <portdnn/conv2d/selector/default_selector.h>
#include <portdnn/conv2d/selector/direct_selector.h>
#include <portdnn/conv2d/selector/im2col_selector.h>
#include <portdnn/conv2d/selector/matmul_selector.h>
#include <portdnn/conv2d/selector/tiled_selector.h>
#include <portdnn/conv2d/selector/winograd_selector.h>
#include <portdnn/conv2d/workspace_size.h>
#include <portdnn/depthwise_conv2d/launch.h>
#include <portdnn/helpers/padding.h>
#include <portdnn/matmul/launch.h>
#include <portdnn/pointwise/launch.h>
#include <portdnn/pooling/launch.h>

#include <cmath>
#include <random>
#include <vector>

#include "../../oracle/oracle.h"
#include "check.h"

using namespace sycldnn;
using conv2d::Conv2DParams;
namespace ct = conv2d::conv_type;

static std::vector<float> iota_data(size_t n, int max_val) {
  std::vector<float> v(n);
  for (size_t i = 0; i < n; ++i) v[i] = static_cast<float>(i % max_val + 1);
  return v;
}
static std::vector<float> uniform_data(size_t n, unsigned seed) {
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> d(-1.f, 1.f);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}

struct DeviceBuffer {
  float* ptr = nullptr;
  size_t n = 0;
  backend::HIPBackend* b;
  DeviceBuffer(backend::HIPBackend& be, std::vector<float> const& host)
      : n(host.size()), b(&be) {
    ptr = be.allocate<float>(n > 0 ? n : 1);
    (void)hipMemcpy(ptr, host.data(), n * sizeof(float), hipMemcpyHostToDevice);
  }
  DeviceBuffer(backend::HIPBackend& be, size_t count) : n(count), b(&be) {
    ptr = be.allocate<float>(n > 0 ? n : 1);
    (void)hipMemset(ptr, 0xff, n * sizeof(float));  // NaN pattern
  }
  ~DeviceBuffer() { b->deallocate(ptr); }
  std::vector<float> host() const {
    std::vector<float> h(n);
    (void)hipMemcpy(h.data(), ptr, n * sizeof(float), hipMemcpyDeviceToHost);
    return h;
  }
};

static bool close(std::vector<float> const& got, std::vector<float> const& ref,
                  bool exact) {
  if (got.size() != ref.size()) return false;
  double sq = 0;
  for (float r : ref) sq += static_cast<double>(r) * r;
  const double scale = std::max(1.0, std::sqrt(sq / std::max<size_t>(1, ref.size())));
  for (size_t i = 0; i < ref.size(); ++i) {
    const double err = std::fabs(static_cast<double>(got[i]) - ref[i]);
    const double tol = exact ? 0.0 : 1e-4 * std::fabs(ref[i]) + 1e-5 * scale;
    if (!(err <= tol)) {
      std::printf("  mismatch at %zu: got %g expected %g\n", i, got[i], ref[i]);
      return false;
    }
  }
  return true;
}

static oracle_params to_oracle(Conv2DParams const& p) {
  return {p.channels, p.features,    p.batch,       p.in_rows,  p.in_cols,
          p.window_rows, p.window_cols, p.stride_rows, p.stride_cols,
          p.out_rows, p.out_cols,    p.pad_rows,    p.pad_cols};
}

template <typename ConvType>
static void test_conv(Conv2DParams const& params, conv2d::Selector& selector,
                      backend::HIPBackend& backend, bool iota) {
  if (selector.select<ConvType>(params) == conv2d::Algorithm::NotSupported)
    return;  // as GTEST_SKIP in the reference fixture
  const auto sizes = conv2d::get_sizes<ConvType>(params);
  const auto in = iota ? iota_data(sizes.input_size, 64)
                       : uniform_data(sizes.input_size, 11);
  const auto fil = iota ? iota_data(sizes.filter_size, 64)
                        : uniform_data(sizes.filter_size, 12);
  DeviceBuffer d_in(backend, in), d_fil(backend, fil);
  DeviceBuffer d_out(backend, sizes.output_size);
  const auto ws = conv2d::query_workspace_size<ConvType>(params, selector);
  DeviceBuffer d_ws(backend, ws.recommended_size);
  auto status = conv2d::launch<float, ConvType>(
      d_in.ptr, d_fil.ptr, d_out.ptr, params, selector, backend, d_ws.ptr,
      ws.recommended_size);
  CHECK(status.status == StatusCode::OK);
  status.event.wait_and_throw();
  std::vector<float> ref(sizes.output_size);
  const oracle_params op = to_oracle(params);
  if (std::is_same<ConvType, ct::Forward>::value)
    oracle_conv2d_forward(in.data(), fil.data(), ref.data(), &op, 1);
  else if (std::is_same<ConvType, ct::InputBackprop>::value)
    oracle_conv2d_input_backprop(in.data(), fil.data(), ref.data(), &op, 1);
  else
    oracle_conv2d_filter_backprop(in.data(), fil.data(), ref.data(), &op, 1);
  const bool ok = close(d_out.host(), ref, iota);
  if (!ok)
    std::printf("  selector %s window %d stride %d C %d K %d\n",
                selector.name(), params.window_rows, params.stride_rows,
                params.channels, params.features);
  CHECK(ok);
}

static Conv2DParams conv_params(int n, int h, int w, int c, int k, int window,
                                int stride, PaddingMode mode) {
  Conv2DParams p{};
  p.channels = c; p.features = k; p.batch = n; p.in_rows = h; p.in_cols = w;
  p.window_rows = p.window_cols = window;
  p.stride_rows = p.stride_cols = stride;
  p.dilation_rows = p.dilation_cols = 1;
  return helpers::add_padding_to(p, mode);
}

static void test_all_conv(backend::HIPBackend& backend) {
  conv2d::DirectSelector direct;
  conv2d::TiledSelector tiled;
  conv2d::Im2colSelector im2col;
  conv2d::WinogradSelector wino;
  conv2d::MatmulSelector mm;
  auto def = conv2d::get_default_selector(backend);
  conv2d::Selector* selectors[] = {&direct, &tiled, &im2col, &wino, &mm,
                                   def.get()};
  const Conv2DParams shapes[] = {
      conv_params(1, 4, 4, 1, 1, 3, 1, PaddingMode::SAME),
      conv_params(3, 5, 6, 2, 4, 3, 2, PaddingMode::VALID),
      conv_params(2, 9, 9, 4, 4, 5, 1, PaddingMode::SAME),
      conv_params(2, 12, 12, 32, 64, 3, 1, PaddingMode::SAME),
      conv_params(2, 8, 8, 64, 256, 1, 1, PaddingMode::VALID),
      conv_params(1, 20, 20, 3, 8, 7, 2, PaddingMode::SAME),
  };
  for (auto* sel : selectors) {
    for (auto const& p : shapes) {
      for (bool iota : {true, false}) {
        test_conv<ct::Forward>(p, *sel, backend, iota);
        test_conv<ct::InputBackprop>(p, *sel, backend, iota);
        test_conv<ct::FilterBackprop>(p, *sel, backend, iota);
      }
    }
  }
}

static void test_depthwise(backend::HIPBackend& backend) {
  depthwise_conv2d::DepthwiseConv2DParams p{};
  p.channels = 32; p.channel_multiplier = 1; p.batch = 2;
  p.in_rows = p.in_cols = 14; p.window_rows = p.window_cols = 3;
  p.stride_rows = p.stride_cols = 2;
  p = helpers::add_padding_to(p, PaddingMode::SAME);
  const auto sizes = depthwise_conv2d::get_sizes<ct::Forward>(p);
  const auto in = uniform_data(sizes.input_size, 3);
  const auto fil = uniform_data(sizes.filter_size, 4);
  DeviceBuffer d_in(backend, in), d_fil(backend, fil);
  DeviceBuffer d_out(backend, sizes.output_size);
  auto st = depthwise_conv2d::launch<float, ct::Forward>(
      d_in.ptr, d_fil.ptr, d_out.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  const oracle_params op = {p.channels, p.channel_multiplier, p.batch,
                            p.in_rows, p.in_cols, p.window_rows, p.window_cols,
                            p.stride_rows, p.stride_cols, p.out_rows,
                            p.out_cols, p.pad_rows, p.pad_cols};
  std::vector<float> ref(sizes.output_size);
  oracle_depthwise_forward(in.data(), fil.data(), ref.data(), &op, 1);
  CHECK(close(d_out.host(), ref, false));
  // gradient w.r.t. the input: dY has the forward output's size
  const auto dy = uniform_data(sizes.output_size, 5);
  DeviceBuffer d_dy(backend, dy), d_dx(backend, sizes.input_size);
  st = depthwise_conv2d::launch<float, ct::InputBackprop>(
      d_dy.ptr, d_fil.ptr, d_dx.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  std::vector<float> ref_dx(sizes.input_size);
  oracle_depthwise_input_backprop(dy.data(), fil.data(), ref_dx.data(), &op, 1);
  CHECK(close(d_dx.host(), ref_dx, false));
}

static void test_pooling(backend::HIPBackend& backend) {
  pooling::PoolingParams p{};
  p.in_rows = p.in_cols = 15; p.window_rows = p.window_cols = 3;
  p.stride_rows = p.stride_cols = 2; p.batch = 2; p.channels = 16;
  p = helpers::add_padding_to(p, PaddingMode::SAME);
  const auto sizes = pooling::get_sizes<pooling::Forward>(p);
  const auto in = uniform_data(sizes.input_size, 7);
  DeviceBuffer d_in(backend, in), d_out(backend, sizes.output_size);
  const oracle_params op = {p.channels, 0, p.batch, p.in_rows, p.in_cols,
                            p.window_rows, p.window_cols, p.stride_rows,
                            p.stride_cols, p.out_rows, p.out_cols, p.pad_rows,
                            p.pad_cols};
  auto st = pooling::launch<float, pooling::Max, pooling::Forward>(
      d_in.ptr, d_out.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  std::vector<float> ref(sizes.output_size);
  oracle_pool_max_forward(in.data(), ref.data(), &op, 0);
  const auto y = d_out.host();
  CHECK(close(y, ref, true));
  // max gradient through the four-pointer overload
  const auto dy = iota_data(sizes.output_size, 97);
  DeviceBuffer d_dy(backend, dy), d_dx(backend, sizes.input_size);
  st = pooling::launch<float, pooling::Max, pooling::Backpropagate>(
      d_in.ptr, d_out.ptr, d_dy.ptr, d_dx.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  std::vector<float> ref_dx(sizes.input_size);
  oracle_pool_max_grad(in.data(), ref.data(), dy.data(), ref_dx.data(), &op, 0);
  CHECK(close(d_dx.host(), ref_dx, true));
  // average forward and gradient
  st = pooling::launch<float, pooling::Average, pooling::Forward>(
      d_in.ptr, d_out.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  oracle_pool_avg_forward(in.data(), ref.data(), &op, 1);
  CHECK(close(d_out.host(), ref, false));
  st = pooling::launch<float, pooling::Average, pooling::Backpropagate>(
      d_dy.ptr, d_dx.ptr, p, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  oracle_pool_avg_grad(dy.data(), ref_dx.data(), &op, 1);
  CHECK(close(d_dx.host(), ref_dx, false));
}

static void test_event_dependencies(backend::HIPBackend& backend) {
  // test/conv2d/conv2d_event_dependencies.cc: a launch given an event must
  // run after it.  Here: conv B consumes conv A's output on another stream.
  hipStream_t other;
  if (hipStreamCreate(&other) != hipSuccess) { CHECK(false); return; }
  backend::HIPBackend backend2(other);
  conv2d::Im2colSelector sel;
  auto p = conv_params(4, 28, 28, 32, 32, 3, 1, PaddingMode::SAME);
  const auto sizes = conv2d::get_sizes<ct::Forward>(p);
  const auto in = uniform_data(sizes.input_size, 21);
  const auto fil = uniform_data(sizes.filter_size, 22);
  DeviceBuffer d_in(backend, in), d_fil(backend, fil);
  DeviceBuffer d_mid(backend, sizes.output_size), d_out(backend, sizes.output_size);
  auto a = conv2d::launch<float, ct::Forward>(d_in.ptr, d_fil.ptr, d_mid.ptr, p,
                                              sel, backend, nullptr, 0);
  CHECK(a.status == StatusCode::OK);
  auto b = conv2d::launch<float, ct::Forward>(d_mid.ptr, d_fil.ptr, d_out.ptr,
                                              p, sel, backend2, nullptr, 0,
                                              {a.event});
  CHECK(b.status == StatusCode::OK);
  b.event.wait_and_throw();
  const oracle_params op = to_oracle(p);
  std::vector<float> mid(sizes.output_size), ref(sizes.output_size);
  oracle_conv2d_forward(in.data(), fil.data(), mid.data(), &op, 1);
  oracle_conv2d_forward(mid.data(), fil.data(), ref.data(), &op, 1);
  CHECK(close(d_out.host(), ref, false));
  (void)hipStreamDestroy(other);
}

// test/matmul/fixture.h:37-76: iota operands and initial output, offset
// pointers, every transpose / beta combination; here also sizes that take the
// matrix-core path (k a multiple of 32) and ones that do not.
template <bool TL, bool TR>
static void test_matmul_case(backend::HIPBackend& backend, int batches, int m,
                             int k, int n, float beta, int offset) {
  const size_t lhs_n = static_cast<size_t>(batches) * m * k + offset;
  const size_t rhs_n = static_cast<size_t>(batches) * k * n + offset;
  const size_t out_n = static_cast<size_t>(batches) * m * n + offset;
  const auto lhs = iota_data(lhs_n, 16), rhs = iota_data(rhs_n, 16);
  const auto out0 = iota_data(out_n, 16);
  DeviceBuffer d_lhs(backend, lhs), d_rhs(backend, rhs), d_out(backend, out0);
  auto status = matmul::launch<float, TL, TR>(
      d_lhs.ptr + offset, d_rhs.ptr + offset, d_out.ptr + offset,
      matmul::MatmulParams{batches, m, k, n, beta}, backend);
  CHECK(status.status == StatusCode::OK);
  status.event.wait_and_throw();
  std::vector<float> ref = out0;
  oracle_matmul(lhs.data() + offset, rhs.data() + offset, ref.data() + offset,
                batches, m, k, n, TL, TR, beta, 1);
  const bool ok = close(d_out.host(), ref, true);
  if (!ok)
    std::printf("  matmul TL %d TR %d batches %d m %d k %d n %d beta %g\n", TL,
                TR, batches, m, k, n, beta);
  CHECK(ok);
}

static void test_matmul(backend::HIPBackend& backend) {
  const int shapes[][4] = {{1, 14, 15, 16}, {3, 16, 14, 15}, {2, 70, 64, 36},
                           {1, 130, 96, 64}, {3, 33, 32, 8}};
  for (auto const& s : shapes) {
    for (float beta : {0.f, 1.f, 2.f}) {
      for (int offset : {0, 8}) {
        test_matmul_case<false, false>(backend, s[0], s[1], s[2], s[3], beta,
                                       offset);
        test_matmul_case<false, true>(backend, s[0], s[1], s[2], s[3], beta,
                                      offset);
        test_matmul_case<true, false>(backend, s[0], s[1], s[2], s[3], beta,
                                      offset);
        test_matmul_case<true, true>(backend, s[0], s[1], s[2], s[3], beta,
                                     offset);
      }
    }
  }
  // internal/matmul/launch.h:66-70: non-positive sizes are invalid parameters
  DeviceBuffer a(backend, 16), b(backend, 16), c(backend, 16);
  CHECK((matmul::launch<float, false, false>(
             a.ptr, b.ptr, c.ptr, matmul::MatmulParams{0, 4, 4, 4, 0.f},
             backend).status == StatusCode::InvalidParameter));
  CHECK((matmul::launch<float, false, false>(
             a.ptr, b.ptr, c.ptr, matmul::MatmulParams{1, 4, -1, 4, 0.f},
             backend).status == StatusCode::InvalidParameter));
  // test/matmul/matmul_event_dependency.cc: the launch waits for its events
  hipStream_t other;
  CHECK(hipStreamCreate(&other) == hipSuccess);
  {
    backend::HIPBackend producer(other);
    const auto x = iota_data(64 * 64, 8);
    DeviceBuffer d_x(backend, x), d_y(backend, 64 * 64), d_z(backend, 64 * 64);
    auto first = matmul::launch<float, false, false>(
        d_x.ptr, d_x.ptr, d_y.ptr, matmul::MatmulParams{1, 64, 64, 64, 0.f},
        producer);
    CHECK(first.status == StatusCode::OK);
    auto second = matmul::launch<float, false, false>(
        d_y.ptr, d_x.ptr, d_z.ptr, matmul::MatmulParams{1, 64, 64, 64, 0.f},
        backend, {first.event});
    CHECK(second.status == StatusCode::OK);
    second.event.wait_and_throw();
    std::vector<float> y(64 * 64, 0.f), z(64 * 64, 0.f);
    oracle_matmul(x.data(), x.data(), y.data(), 1, 64, 64, 64, 0, 0, 0.f, 1);
    oracle_matmul(y.data(), x.data(), z.data(), 1, 64, 64, 64, 0, 0, 0.f, 1);
    CHECK(close(d_z.host(), z, true));
  }
  (void)hipStreamDestroy(other);
}

// test/pointwise/pointwise_fixture.h:37-70 (forward) and :72-137 (gradient),
// test/binaryop/fixture.h:37-76.
static void test_elementwise(backend::HIPBackend& backend) {
  const size_t n = 4099;
  std::vector<float> x(n);
  for (size_t i = 0; i < n; ++i)
    x[i] = static_cast<float>(static_cast<long>(i % 17) - 8);
  DeviceBuffer d_x(backend, x), d_y(backend, n), d_g(backend, n);
  auto st = pointwise::launch<float, pointwise::Relu, pointwise::Forward>(
      d_x.ptr, d_y.ptr, n, backend);
  CHECK(st.status == StatusCode::OK);
  auto gr = pointwise::launch<float, pointwise::Relu, pointwise::Gradient>(
      d_y.ptr, d_x.ptr, d_g.ptr, n, backend, {st.event});
  CHECK(gr.status == StatusCode::OK);
  gr.event.wait_and_throw();
  std::vector<float> y(n), g(n);
  CHECK(oracle_pointwise_forward(ORACLE_RELU, x.data(), y.data(), n) == 0);
  CHECK(oracle_pointwise_grad(ORACLE_RELU, y.data(), x.data(), g.data(), n) ==
        0);
  CHECK(close(d_y.host(), y, true));
  CHECK(close(d_g.host(), g, true));
  CHECK((pointwise::launch<float, pointwise::Tanh, pointwise::Forward>(
             d_x.ptr, d_y.ptr, 0, backend).status ==
         StatusCode::InvalidParameter));

  // bias add over an NHWC tensor, then a general broadcast
  const std::vector<int> t_dims = {2, 5, 7, 12}, b_dims = {12};
  const auto t = iota_data(2 * 5 * 7 * 12, 9), b = iota_data(12, 5);
  DeviceBuffer d_t(backend, t), d_b(backend, b), d_o(backend, t.size());
  binaryop::BinaryParams params{t_dims, b_dims};
  auto add = binaryop::launch<float, binaryop::Add>(d_t.ptr, d_b.ptr, d_o.ptr,
                                                    params, backend);
  CHECK(add.status == StatusCode::OK);
  add.event.wait_and_throw();
  std::vector<float> ref(t.size());
  CHECK(oracle_binaryop(ORACLE_ADD, t.data(), b.data(), ref.data(),
                        t_dims.data(), 4, b_dims.data(), 1) == 0);
  CHECK(close(d_o.host(), ref, true));
  const std::vector<int> l_dims = {3, 1, 4}, r_dims = {2, 1, 5, 1};
  const auto l = iota_data(12, 7), r = iota_data(10, 3);
  DeviceBuffer d_l(backend, l), d_r(backend, r), d_q(backend, 2 * 3 * 5 * 4);
  auto mul = binaryop::launch<float, binaryop::Mul>(
      d_l.ptr, d_r.ptr, d_q.ptr, binaryop::BinaryParams{l_dims, r_dims},
      backend);
  CHECK(mul.status == StatusCode::OK);
  mul.event.wait_and_throw();
  std::vector<float> ref2(2 * 3 * 5 * 4);
  CHECK(oracle_binaryop(ORACLE_MUL, l.data(), r.data(), ref2.data(),
                        l_dims.data(), 3, r_dims.data(), 4) == 0);
  CHECK(close(d_q.host(), ref2, true));
  // internal/binaryop/launch.h:52-56: shapes that do not broadcast
  CHECK((binaryop::launch<float, binaryop::Sub>(
             d_l.ptr, d_r.ptr, d_q.ptr, binaryop::BinaryParams{{3, 4}, {5, 4}},
             backend).status == StatusCode::InvalidParameter));
}

// test/compat/conv2d_forward_compat.cc:77-172 (fixture) with its hand-written
// cases :174-446: operands and the initial output are 1,2,3,... (max 2048).
static void compat_case(compat::SNNHandle& handle, std::vector<int> in_sizes,
                        std::vector<int> filt_sizes, std::vector<int> conv,
                        std::vector<float> expect, DataFormat format,
                        conv2d::Algorithm algo, float alpha, float beta,
                        StatusCode want = StatusCode::OK, int groups = 1) {
  using namespace compat;
  backend::HIPBackend& backend = handle.getBackend();
  TensorDescriptor x_desc, y_desc;
  FilterDescriptor w_desc;
  ConvolutionDescriptor c_desc;
  CHECK(x_desc.set4d(format, in_sizes[0], in_sizes[1], in_sizes[2],
                     in_sizes[3]) == StatusCode::OK);
  CHECK(w_desc.set4d(format, filt_sizes[0], filt_sizes[1], filt_sizes[2],
                     filt_sizes[3]) == StatusCode::OK);
  CHECK(c_desc.set2d(conv[0], conv[1], conv[2], conv[3], conv[4], conv[5]) ==
        StatusCode::OK);
  if (groups > 1) CHECK(setConvolutionGroupCount(c_desc, groups) == StatusCode::OK);
  int n, c, h, w;
  CHECK(getConvolution2dForwardOutputDim(c_desc, x_desc, w_desc, &n, &c, &h,
                                         &w) == StatusCode::OK);
  CHECK(y_desc.set4d(format, n, c, h, w) == StatusCode::OK);
  DeviceBuffer d_x(backend, iota_data(x_desc.getSize(), 2048));
  DeviceBuffer d_w(backend, iota_data(w_desc.getSize(), 2048));
  DeviceBuffer d_y(backend, iota_data(y_desc.getSize(), 2048));
  SNNStatus st = convolutionForward(handle, &alpha, x_desc, d_x.ptr, w_desc,
                                    d_w.ptr, c_desc, algo, nullptr, 0, &beta,
                                    y_desc, d_y.ptr);
  CHECK(st.status == want);
  if (want != StatusCode::OK) return;
  st.event.wait_and_throw();
  const bool ok = close(d_y.host(), expect, true);
  if (!ok) std::printf("  compat case alpha %g beta %g\n", alpha, beta);
  CHECK(ok);
}

// conv + bias + ReLU in one launch against the reference's three.
static void test_bias_activation(backend::HIPBackend& backend) {
  Conv2DParams p{};
  p.channels = 64; p.features = 96; p.batch = 2;
  p.in_rows = p.in_cols = 14;
  p.window_rows = p.window_cols = 3;
  p.stride_rows = p.stride_cols = 1;
  p = helpers::add_padding_to(p, PaddingMode::SAME);
  const auto sizes = conv2d::get_sizes<ct::Forward>(p);
  const auto x = uniform_data(sizes.input_size, 21);
  const auto w = uniform_data(sizes.filter_size, 22);
  const auto b = uniform_data(p.features, 23);
  DeviceBuffer d_x(backend, x), d_w(backend, w), d_b(backend, b);
  DeviceBuffer d_fused(backend, sizes.output_size),
      d_three(backend, sizes.output_size);
  conv2d::WinogradSelector wino;
  const auto ws = conv2d::query_workspace_size<ct::Forward>(p, wino);
  DeviceBuffer d_ws(backend, ws.recommended_size);
  auto st = conv2d::launch_forward_bias_activation<float>(
      d_x.ptr, d_w.ptr, d_b.ptr, d_fused.ptr, p, wino, backend, d_ws.ptr,
      ws.recommended_size, conv2d::Activation::Relu);
  CHECK(st.status == StatusCode::OK);
  st = conv2d::launch<float, ct::Forward>(d_x.ptr, d_w.ptr, d_three.ptr, p,
                                          wino, backend, d_ws.ptr,
                                          ws.recommended_size);
  CHECK(st.status == StatusCode::OK);
  st = binaryop::launch<float, binaryop::Add>(
      d_three.ptr, d_b.ptr, d_three.ptr,
      binaryop::BinaryParams{{p.batch, p.out_rows, p.out_cols, p.features},
                             {p.features}},
      backend);
  CHECK(st.status == StatusCode::OK);
  st = pointwise::launch<float, pointwise::Relu, pointwise::Forward>(
      d_three.ptr, d_three.ptr, sizes.output_size, backend);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  CHECK(close(d_fused.host(), d_three.host(), true));
}

// The two-call form: prepare_filter once, launch_prepared many times; the
// one-call launch in between must not depend on what the workspace holds.
static void test_prepared_filter(backend::HIPBackend& backend) {
  Conv2DParams p{};
  p.channels = 64; p.features = 64; p.batch = 3;
  p.in_rows = p.in_cols = 14;
  p.window_rows = p.window_cols = 3;
  p.stride_rows = p.stride_cols = 1;
  p = helpers::add_padding_to(p, PaddingMode::SAME);
  const auto sizes = conv2d::get_sizes<ct::Forward>(p);
  const auto x = uniform_data(sizes.input_size, 31);
  const auto w = uniform_data(sizes.filter_size, 32);
  DeviceBuffer d_x(backend, x), d_w(backend, w);
  DeviceBuffer d_one(backend, sizes.output_size),
      d_two(backend, sizes.output_size);
  std::unique_ptr<conv2d::Selector> def(new conv2d::WinogradSelector());
  const auto ws = conv2d::query_workspace_size<float, ct::Forward>(p, *def);
  CHECK(ws.recommended_size >= ws.required_size && ws.required_size > 0);
  DeviceBuffer d_ws(backend, ws.recommended_size);
  auto st = conv2d::launch<float, ct::Forward>(d_x.ptr, d_w.ptr, d_one.ptr, p,
                                               *def, backend, d_ws.ptr,
                                               ws.recommended_size);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  // garbage in the workspace, then prepare + two prepared launches
  (void)hipMemset(d_ws.ptr, 0xff, ws.recommended_size * sizeof(float));
  st = conv2d::prepare_filter<float, ct::Forward>(
      d_w.ptr, p, *def, backend, d_ws.ptr, ws.recommended_size);
  CHECK(st.status == StatusCode::OK);
  for (int rep = 0; rep < 2; ++rep) {
    st = conv2d::launch_prepared<float, ct::Forward>(
        d_x.ptr, d_w.ptr, d_two.ptr, p, *def, backend, d_ws.ptr,
        ws.recommended_size);
    CHECK(st.status == StatusCode::OK);
  }
  st.event.wait_and_throw();
  CHECK(close(d_two.host(), d_one.host(), true));
  // an algorithm with nothing to prepare takes both calls as well
  conv2d::Im2colSelector im2col;
  st = conv2d::prepare_filter<float, ct::Forward>(d_w.ptr, p, im2col, backend,
                                                  d_ws.ptr, ws.recommended_size);
  CHECK(st.status == StatusCode::OK);
  st = conv2d::launch_prepared<float, ct::Forward>(
      d_x.ptr, d_w.ptr, d_two.ptr, p, im2col, backend, d_ws.ptr,
      ws.recommended_size);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  CHECK(close(d_two.host(), d_one.host(), false));
}

static void test_compat(hipStream_t stream) {
  using namespace compat;
  using A = conv2d::Algorithm;
  // test/compat/conv2d_forward_compat.cc:25-67
  ConvolutionDescriptor desc;
  CHECK(setConvolution2dDescriptor(desc, 1, 2, 3, 4, 1, 1,
                                   ConvolutionMode::CROSS_CORRELATION) ==
        StatusCode::OK);
  CHECK(desc.getPadH() == 1 && desc.getPadW() == 2 && desc.getStrideH() == 3 &&
        desc.getStrideW() == 4 && desc.getDilationH() == 1 &&
        desc.getMode() == ConvolutionMode::CROSS_CORRELATION);
  CHECK(desc.set2d(-1, 0, 1, 1, 1, 1) == StatusCode::InvalidParameter);
  CHECK(desc.set2d(0, 0, 1, 1, 1, 1, ConvolutionMode::CONVOLUTION) ==
        StatusCode::InvalidParameter);
  setConvolutionGroupCount(desc, 5);
  CHECK(desc.getGroupCount() == 5);

  SNNHandle handle;
  CHECK(SNNCreate(handle, stream) == StatusCode::OK);
  const DataFormat nhwc = DataFormat::NHWC, nchw = DataFormat::NCHW;
  const std::vector<int> unit = {0, 0, 1, 1, 1, 1};
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {348, 393, 528, 573},
              nhwc, A::Direct, 1.f, 0.f);
  compat_case(handle, {2, 3, 1, 1}, {1, 3, 1, 1}, unit, {14, 32}, nhwc,
              A::Direct, 1.f, 0.f);
  compat_case(handle, {1, 1, 1, 1}, {1, 1, 3, 3}, {1, 1, 1, 1, 1, 1}, {5},
              nhwc, A::Direct, 1.f, 0.f);
  compat_case(handle, {1, 3, 1, 1}, {1, 3, 3, 3}, {1, 1, 1, 1, 1, 1}, {86},
              nhwc, A::Direct, 1.f, 0.f);
  compat_case(handle, {1, 1, 5, 5}, {1, 1, 3, 3}, {0, 0, 2, 2, 1, 1},
              {411, 501, 861, 951}, nchw, A::Direct, 1.f, 0.f);
  compat_case(handle, {1, 1, 11, 11}, {2, 1, 7, 7}, {2, 2, 4, 4, 1, 1},
              {48425., 49050., 72800., 73780., 55075., 55850., 125230.,
               127260., 177037., 180026., 126980., 129220., 91975., 94250.,
               126210., 129500., 87825., 90250.},
              nhwc, A::Im2col, 1.f, 0.f);
  // alpha / beta, :285-446
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {696, 786, 1056, 1146},
              nhwc, A::Direct, 2.f, 0.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {0, 0, 0, 0}, nhwc,
              A::Direct, 0.f, 0.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit,
              {-696, -786, -1056, -1146}, nhwc, A::Direct, -2.f, 0.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {349, 395, 531, 577},
              nhwc, A::Direct, 1.f, 1.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {1, 2, 3, 4}, nhwc,
              A::Direct, 0.f, 1.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {2, 4, 6, 8}, nhwc,
              A::Direct, 0.f, 2.f);
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit, {-2, -4, -6, -8}, nhwc,
              A::Direct, 0.f, -2.f);
  // both factors at once: 3 * conv - 2 * prior
  compat_case(handle, {1, 1, 4, 4}, {1, 1, 3, 3}, unit,
              {3 * 348 - 2, 3 * 393 - 4, 3 * 528 - 6, 3 * 573 - 8}, nhwc,
              A::Direct, 3.f, -2.f);
  // grouped convolutions are not provided
  compat_case(handle, {1, 2, 5, 5}, {2, 1, 2, 2}, unit, {}, nhwc, A::Im2col,
              1.f, 0.f, StatusCode::InvalidAlgorithm, 2);
  // NCHW runs on Direct only (internal/conv2d/launch.h:191-194)
  compat_case(handle, {1, 1, 5, 5}, {1, 1, 3, 3}, {0, 0, 2, 2, 1, 1}, {}, nchw,
              A::Im2col, 1.f, 0.f, StatusCode::InvalidAlgorithm);

  // workspace size in bytes = recommended elements * sizeof(float)
  TensorDescriptor x_desc, y_desc;
  FilterDescriptor w_desc;
  ConvolutionDescriptor c_desc;
  x_desc.set4d(nhwc, 2, 64, 28, 28);
  w_desc.set4d(nhwc, 64, 64, 3, 3);
  c_desc.set2d(1, 1, 1, 1, 1, 1);
  int n, c, h, w;
  getConvolution2dForwardOutputDim(c_desc, x_desc, w_desc, &n, &c, &h, &w);
  CHECK(n == 2 && c == 64 && h == 28 && w == 28);
  y_desc.set4d(nhwc, n, c, h, w);
  size_t bytes = 0;
  CHECK(getConvolutionForwardWorkspaceSize(handle, x_desc, w_desc, c_desc,
                                           y_desc, A::Winograd, &bytes) ==
        StatusCode::OK);
  conv2d::WinogradSelector wino;
  const auto ws = conv2d::query_workspace_size<ct::Forward>(
      compat::internal::descToSnnParams(x_desc, y_desc, w_desc, c_desc), wino);
  CHECK(bytes == ws.recommended_size * sizeof(float) && bytes > 0);

  // backward data / filter against the oracle, NHWC, with a blend
  const auto x = uniform_data(x_desc.getSize(), 11);
  const auto wt = uniform_data(w_desc.getSize(), 12);
  const auto dy = uniform_data(y_desc.getSize(), 13);
  backend::HIPBackend& backend = handle.getBackend();
  DeviceBuffer d_x(backend, x), d_w(backend, wt), d_dy(backend, dy);
  const auto dx0 = uniform_data(x_desc.getSize(), 14);
  const auto dw0 = uniform_data(w_desc.getSize(), 15);
  DeviceBuffer d_dx(backend, dx0), d_dw(backend, dw0);
  const float alpha = 0.5f, beta = 2.f;
  auto st = convolutionBackwardData(handle, &alpha, w_desc, d_w.ptr, y_desc,
                                    d_dy.ptr, c_desc, A::Im2col, nullptr, 0,
                                    &beta, x_desc, d_dx.ptr);
  CHECK(st.status == StatusCode::OK);
  st = convolutionBackwardFilter(handle, &alpha, x_desc, d_x.ptr, y_desc,
                                 d_dy.ptr, c_desc, A::Im2col, nullptr, 0, &beta,
                                 w_desc, d_dw.ptr);
  CHECK(st.status == StatusCode::OK);
  st.event.wait_and_throw();
  oracle_params op{64, 64, 2, 28, 28, 3, 3, 1, 1, 28, 28, 1, 1};
  std::vector<float> dx(x.size()), dw(wt.size());
  oracle_conv2d_input_backprop(dy.data(), wt.data(), dx.data(), &op, 1);
  oracle_conv2d_filter_backprop(x.data(), dy.data(), dw.data(), &op, 1);
  for (size_t i = 0; i < dx.size(); ++i) dx[i] = alpha * dx[i] + beta * dx0[i];
  for (size_t i = 0; i < dw.size(); ++i) dw[i] = alpha * dw[i] + beta * dw0[i];
  CHECK(close(d_dx.host(), dx, false));
  CHECK(close(d_dw.host(), dw, false));
}

int main() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    std::printf("gpu_api_test: no GPU\n");
    return 2;
  }
  hipStream_t stream;
  if (hipStreamCreate(&stream) != hipSuccess) return 2;
  {
    backend::HIPBackend backend(stream);
    test_all_conv(backend);
    test_depthwise(backend);
    test_pooling(backend);
    test_event_dependencies(backend);
    test_matmul(backend);
    test_elementwise(backend);
    test_bias_activation(backend);
    test_prepared_filter(backend);
  }
  test_compat(stream);
  (void)hipStreamDestroy(stream);
  return report("gpu_api_test");
}
