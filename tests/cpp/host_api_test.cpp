// Host-side test of the sycldnn:: drop-in headers: runs without a GPU.
// Mirrors the reference's host tests: test/helpers/padding.cc,
// test/conv2d/workspace_size.cc, test/conv2d/default_selector.cc and the
// parameter validation of include/portdnn/internal/conv2d/launch.h:42-97.
#include <portdnn/backend/hip_backend.h>
#include <portdnn/conv2d/launch.h>
#include <portdnn/conv2d/selector/default_selector.h>
#include <portdnn/conv2d/selector/direct_selector.h>
#include <portdnn/conv2d/selector/im2col_selector.h>
#include <portdnn/conv2d/selector/matmul_selector.h>
#include <portdnn/conv2d/selector/tiled_selector.h>
#include <portdnn/conv2d/selector/winograd_selector.h>
#include <portdnn/conv2d/sizes.h>
#include <portdnn/conv2d/workspace_size.h>
#include <portdnn/depthwise_conv2d/launch.h>
#include <portdnn/depthwise_conv2d/sizes.h>
#include <portdnn/helpers/padding.h>
#include <portdnn/matmul/launch.h>
#include <portdnn/matmul/params.h>
#include <portdnn/pooling/launch.h>
#include <portdnn/pooling/sizes.h>

#include "check.h"

using namespace sycldnn;
using conv2d::Algorithm;
using conv2d::Conv2DParams;
namespace ct = conv2d::conv_type;

static Conv2DParams make(int window, int stride, int size, int channels,
                         int features, int batch, PaddingMode mode) {
  Conv2DParams p{};
  p.window_rows = p.window_cols = window;
  p.stride_rows = p.stride_cols = stride;
  p.in_rows = p.in_cols = size;
  p.channels = channels;
  p.features = features;
  p.batch = batch;
  p.dilation_rows = p.dilation_cols = 1;
  return helpers::add_padding_to(p, mode);
}

static void test_padding() {
  // the shapes of the benchmark layers
  auto a = helpers::calculate_padding(56, 3, 1, PaddingMode::SAME);
  CHECK_EQ(a.padding, 1); CHECK_EQ(a.output, 56);
  a = helpers::calculate_padding(112, 3, 2, PaddingMode::SAME);
  CHECK_EQ(a.padding, 0); CHECK_EQ(a.output, 56);
  a = helpers::calculate_padding(224, 7, 2, PaddingMode::SAME);
  CHECK_EQ(a.padding, 2); CHECK_EQ(a.output, 112);
  a = helpers::calculate_padding(7, 7, 1, PaddingMode::VALID);
  CHECK_EQ(a.padding, 0); CHECK_EQ(a.output, 1);
  // test/helpers/padding.cc SameWindow3Stride2 / SameWindow3Stride3 rows
  const int in[8] = {3, 4, 5, 6, 7, 8, 9, 10};
  const int pad2[8] = {1, 0, 1, 0, 1, 0, 1, 0}, out2[8] = {2, 2, 3, 3, 4, 4, 5, 5};
  const int pad3[8] = {0, 1, 0, 0, 1, 0, 0, 1}, out3[8] = {1, 2, 2, 2, 3, 3, 3, 4};
  for (int i = 0; i < 8; ++i) {
    auto r = helpers::calculate_padding(in[i], 3, 2, PaddingMode::SAME);
    CHECK_EQ(r.padding, pad2[i]); CHECK_EQ(r.output, out2[i]);
    r = helpers::calculate_padding(in[i], 3, 3, PaddingMode::SAME);
    CHECK_EQ(r.padding, pad3[i]); CHECK_EQ(r.output, out3[i]);
  }
  CHECK_EQ(helpers::round_ratio_up(7, 2), 4);
  CHECK_EQ(helpers::round_ratio_up(-3, 2), -1);
  CHECK_EQ(helpers::round_ratio_up_above_zero(-3, 2), 0);
  CHECK_EQ(helpers::round_up_to_nearest_multiple(13, 4), 16);
}

static void test_sizes() {
  auto p = make(3, 2, 9, 5, 7, 3, PaddingMode::SAME);
  CHECK_EQ(p.out_rows, 5);
  auto f = conv2d::get_sizes<ct::Forward>(p);
  CHECK_EQ(f.input_size, 3 * 9 * 9 * 5);
  CHECK_EQ(f.filter_size, 3 * 3 * 5 * 7);
  CHECK_EQ(f.output_size, 3 * 5 * 5 * 7);
  auto i = conv2d::get_sizes<ct::InputBackprop>(p);
  CHECK_EQ(i.input_size, f.output_size);
  CHECK_EQ(i.output_size, f.input_size);
  auto b = conv2d::get_sizes<ct::FilterBackprop>(p);
  CHECK_EQ(b.input_size, f.input_size);
  CHECK_EQ(b.filter_size, f.output_size);
  CHECK_EQ(b.output_size, f.filter_size);

  depthwise_conv2d::DepthwiseConv2DParams d{};
  d.channels = 6; d.channel_multiplier = 2; d.batch = 2;
  d.in_rows = d.in_cols = 8; d.window_rows = d.window_cols = 3;
  d.stride_rows = d.stride_cols = 1;
  d = helpers::add_padding_to(d, PaddingMode::VALID);
  auto ds = depthwise_conv2d::get_sizes<ct::Forward>(d);
  CHECK_EQ(ds.output_size, 2 * 6 * 6 * 12);
  CHECK_EQ(ds.filter_size, 3 * 3 * 6 * 2);

  pooling::PoolingParams q{};
  q.in_rows = q.in_cols = 112; q.window_rows = q.window_cols = 3;
  q.stride_rows = q.stride_cols = 2; q.batch = 32; q.channels = 64;
  q = helpers::add_padding_to(q, PaddingMode::SAME);
  CHECK_EQ(q.out_rows, 56); CHECK_EQ(q.pad_rows, 0);
  CHECK_EQ(pooling::get_sizes<pooling::Forward>(q).output_size,
           32 * 56 * 56 * 64);
  CHECK_EQ(pooling::get_sizes<pooling::Backpropagate>(q).output_size,
           32 * 112 * 112 * 64);
}

static void test_selectors() {
  conv2d::TiledSelector tiled;
  conv2d::WinogradSelector wino;
  conv2d::MatmulSelector mm;
  conv2d::DirectSelector direct;
  conv2d::Im2colSelector im2col;
  auto p33 = make(3, 1, 56, 64, 64, 1, PaddingMode::SAME);
  CHECK(tiled.select<ct::Forward>(p33) == Algorithm::Tiled);
  CHECK(tiled.select<ct::InputBackprop>(p33) == Algorithm::NotSupported);
  CHECK(tiled.select<ct::FilterBackprop>(p33) == Algorithm::NotSupported);
  CHECK(wino.select<ct::Forward>(p33) == Algorithm::Winograd);
  CHECK(wino.select<ct::FilterBackprop>(p33) == Algorithm::Winograd);
  CHECK(mm.select<ct::Forward>(p33) == Algorithm::NotSupported);
  CHECK(direct.select<ct::Forward>(p33) == Algorithm::Direct);
  CHECK(im2col.select<ct::FilterBackprop>(p33) == Algorithm::Im2col);
  auto p72 = make(7, 2, 224, 3, 64, 1, PaddingMode::SAME);
  CHECK(tiled.select<ct::Forward>(p72) == Algorithm::NotSupported);
  CHECK(wino.select<ct::Forward>(p72) == Algorithm::NotSupported);
  auto p11 = make(1, 1, 56, 64, 256, 1, PaddingMode::VALID);
  CHECK(mm.select<ct::Forward>(p11) == Algorithm::Matmul);
  CHECK(mm.select<ct::InputBackprop>(p11) == Algorithm::Matmul);
  // test/conv2d/default_selector.cc:73-98: the default is always launchable
  auto def = conv2d::get_default_selector();
  for (auto const& p : {p33, p72, p11}) {
    CHECK(def->select<ct::Forward>(p) != Algorithm::NotSupported);
    CHECK(def->select<ct::InputBackprop>(p) != Algorithm::NotSupported);
    CHECK(def->select<ct::FilterBackprop>(p) != Algorithm::NotSupported);
  }
  CHECK(def->name() != nullptr);
}

static void test_workspace() {
  // test/conv2d/workspace_size.cc:52-160 (VGG layer 1)
  auto p = make(3, 1, 224, 64, 64, 32, PaddingMode::SAME);
  conv2d::DirectSelector direct;
  conv2d::TiledSelector tiled;
  conv2d::Im2colSelector im2col;
  conv2d::WinogradSelector wino;
  auto z = conv2d::query_workspace_size<ct::Forward>(p, direct);
  CHECK_EQ(z.required_size, 0); CHECK_EQ(z.recommended_size, 0);
  z = conv2d::query_workspace_size<ct::FilterBackprop>(p, tiled);
  CHECK_EQ(z.required_size, 0); CHECK_EQ(z.recommended_size, 0);
  const size_t tiles = 224u * 224u, tile = 3u * 3u * 64u, fil = 9u * 64u * 64u;
  auto w = conv2d::query_workspace_size<ct::Forward>(p, im2col);
  CHECK(w.required_size >= tiles * tile);
  CHECK(w.recommended_size >= 32u * tiles * tile);
  w = conv2d::query_workspace_size<ct::InputBackprop>(p, im2col);
  CHECK(w.required_size >= tiles * tile + fil);
  CHECK(w.recommended_size >= 32u * tiles * tile + fil);
  w = conv2d::query_workspace_size<ct::FilterBackprop>(p, im2col);
  CHECK(w.required_size >= tiles * tile);
  const size_t t = 112u * 112u * 64u, f = 64u * 64u;
  w = conv2d::query_workspace_size<ct::Forward>(p, wino);
  CHECK(w.required_size >= 16u * (t + f + t));
  CHECK(w.recommended_size >= 16u * (32u * (t + t) + f));
  w = conv2d::query_workspace_size<ct::InputBackprop>(p, wino);
  CHECK(w.required_size >= 16u * (t + f + t));
  // The reference's bound for the filter gradient (16 * (t + t + f), sized for
  // its three transform buffers) is not kept: this library's kernel for that
  // direction stores no transformed tensors, and the query reports what a
  // launch uses.
  w = conv2d::query_workspace_size<ct::FilterBackprop>(p, wino);
  CHECK(w.required_size <= w.recommended_size);
}

// The element type as a template argument: half never gets Winograd and
// needs no workspace (not in portDNN, whose queries do not know the type).
static void test_typed_selector_and_workspace() {
  // (a host compiler need not know _Float16: the headers take any two-byte
  // element type for binary16)
  using half_t = unsigned short;
  auto p33 = make(3, 1, 56, 64, 64, 128, PaddingMode::SAME);
  auto p11 = make(1, 1, 56, 64, 256, 128, PaddingMode::VALID);
  auto for_float = conv2d::get_default_selector_for<float>();
  auto for_half = conv2d::get_default_selector_for<half_t>();
  CHECK(for_float->select<ct::Forward>(p33) == Algorithm::Winograd);
  CHECK(for_half->select<ct::Forward>(p33) != Algorithm::Winograd);
  CHECK(for_half->select<ct::Forward>(p33) != Algorithm::NotSupported);
  CHECK(for_half->select<ct::InputBackprop>(p33) != Algorithm::Winograd);
  CHECK(for_half->select<ct::FilterBackprop>(p33) != Algorithm::Winograd);
  CHECK(for_half->select<ct::Forward>(p11) == Algorithm::Matmul);
  auto f = conv2d::query_workspace_size<float, ct::Forward>(p33, *for_float);
  auto untyped = conv2d::query_workspace_size<ct::Forward>(p33, *for_float);
  CHECK_EQ(f.required_size, untyped.required_size);
  CHECK_EQ(f.recommended_size, untyped.recommended_size);
  CHECK(f.required_size > 0);
  auto h = conv2d::query_workspace_size<half_t, ct::Forward>(p33, *for_half);
  CHECK_EQ(h.required_size, 0);
  CHECK(h.recommended_size >= 9u * 64u * 64u);  // the re-laid-out filter
  conv2d::WinogradSelector wino;  // the tag on half data: no fp32 buffers
  h = conv2d::query_workspace_size<half_t, ct::Forward>(p33, wino);
  CHECK_EQ(h.required_size, 0);
  CHECK(h.recommended_size < f.required_size);
}

static void test_status_codes() {
  // No GPU work is enqueued by any of these: every launch fails validation.
  backend::HIPBackend backend;
  conv2d::DirectSelector direct;
  conv2d::WinogradSelector wino;
  conv2d::TiledSelector tiled;
  float* fake = reinterpret_cast<float*>(0x1000);
  auto ok = make(3, 1, 8, 4, 4, 2, PaddingMode::SAME);
  auto bad = ok;
  bad.batch = 0;
  auto st = conv2d::launch<float, ct::Forward>(fake, fake, fake, bad, direct,
                                               backend, nullptr, 0);
  CHECK(st.status == StatusCode::InvalidParameter);
  bad = ok;
  bad.dilation_rows = 2;
  st = conv2d::launch<float, ct::Forward>(fake, fake, fake, bad, direct,
                                          backend, nullptr, 0);
  CHECK(st.status == StatusCode::InvalidParameter);
  // Winograd never allocates its own scratch
  st = conv2d::launch<float, ct::Forward>(fake, fake, fake, ok, wino, backend,
                                          nullptr, 0);
  CHECK(st.status == StatusCode::InsufficientWorkspace);
  // a selector answering NotSupported
  st = conv2d::launch<float, ct::InputBackprop>(fake, fake, fake, ok, tiled,
                                                backend, nullptr, 0);
  CHECK(st.status == StatusCode::InvalidAlgorithm);
  auto huge = make(1, 1, 1024, 4, 4, 4096, PaddingMode::VALID);
  st = conv2d::launch<float, ct::Forward>(fake, fake, fake, huge, direct,
                                          backend, nullptr, 0);
  CHECK(st.status == StatusCode::IndexExceeded);

  depthwise_conv2d::DepthwiseConv2DParams d{};
  d.channels = 4; d.channel_multiplier = 0; d.batch = 1;
  d.in_rows = d.in_cols = 8; d.window_rows = d.window_cols = 3;
  d.stride_rows = d.stride_cols = 1;
  d = helpers::add_padding_to(d, PaddingMode::SAME);
  st = depthwise_conv2d::launch<float, ct::Forward>(fake, fake, fake, d,
                                                    backend);
  CHECK(st.status == StatusCode::InvalidParameter);

  pooling::PoolingParams q{};
  q.in_rows = q.in_cols = 8; q.window_rows = q.window_cols = 3;
  q.stride_rows = 2; q.stride_cols = 0; q.batch = 1; q.channels = 4;
  q.out_rows = q.out_cols = 4;
  st = pooling::launch<float, pooling::Max, pooling::Forward>(fake, fake, q,
                                                              backend);
  CHECK(st.status == StatusCode::InvalidParameter);
  st = pooling::launch<float, pooling::Max, pooling::Backpropagate>(
      fake, fake, fake, fake, q, backend);
  CHECK(st.status == StatusCode::InvalidParameter);

  // internal/matmul/launch.h:66-70; defaults of matmul/params.h:52
  matmul::MatmulParams mp{1, 4, 0, 4, 0.f};
  CHECK(mp.batch_type == sycldnn::BatchFormat::STRIDED);
  st = matmul::launch<float, false, true>(fake, fake, fake, mp, backend);
  CHECK(st.status == StatusCode::InvalidParameter);
  mp.k = 4;
  mp.batch_type = sycldnn::BatchFormat::INTERLEAVED;
  st = matmul::launch<float, false, false>(fake, fake, fake, mp, backend);
  CHECK(st.status == StatusCode::InvalidAlgorithm);
}

int main() {
  test_padding();
  test_sizes();
  test_selectors();
  test_workspace();
  test_typed_selector_and_workspace();
  test_status_codes();
  return report("host_api_test");
}
