// Test driver for the C++ host side (mograd_amd/host/mograd_exec.hpp).
//
//   selftest rules      prints "OP_TYPE exec_name" per rule of the table; touches no GPU
//   selftest run        runs the cases below on GPU 0 through the exec functions and prints
//                       "PASS <case>" / "FAIL <case>: <why>"; exit status 1 if any failed
//
// The cases are the reference's own golden vectors and closed forms for the path (each cites
// its test), products of small integers that are exact in fp32, and the reference's error
// conditions.  Expected values are the literal numbers of the reference's assertions or plain
// host loops over the same integers; nothing here comes from the library under test.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "mograd_exec.hpp"

using namespace mograd;

namespace {

int g_failed = 0;

void report(const std::string& name, const std::string& why) {
  if (why.empty()) {
    std::printf("PASS %s\n", name.c_str());
  } else {
    std::printf("FAIL %s: %s\n", name.c_str(), why.c_str());
    ++g_failed;
  }
  std::fflush(stdout);
}

void run_case(const std::string& name, const std::function<std::string()>& body) {
  std::printf("CASE %s\n", name.c_str());
  std::fflush(stdout);
  try {
    report(name, body());
  } catch (const Error& e) {
    report(name, std::string("raised: ") + e.what());
  }
}

AnyBuffer upload(Device& dev, const std::vector<float>& v) { return AnyBuffer::from_host(dev, v.data(), static_cast<int64_t>(v.size()), float32); }

std::vector<float> download(const AnyBuffer& b) {
  std::vector<float> out(static_cast<size_t>(b.numel()));
  b.to_host(out.data());
  return out;
}

std::string close_to(const std::vector<float>& got, const std::vector<double>& want, double atol, const char* what) {
  if (got.size() != want.size()) return std::string(what) + ": size " + std::to_string(got.size()) + " vs " + std::to_string(want.size());
  for (size_t i = 0; i < got.size(); ++i)
    if (!(std::fabs(got[i] - want[i]) <= atol))
      return std::string(what) + "[" + std::to_string(i) + "] = " + std::to_string(got[i]) + ", want " + std::to_string(want[i]);
  return "";
}

OpRef node(const char* op, const Layout& layout, std::vector<OpRef> srcs, std::map<std::string, double> attrs = {}) {
  return OpRef{op, layout, float32, std::move(srcs), std::move(attrs)};
}

// ---- LayerNorm goldens --------------------------------------------------------------------------

std::string ln_fwd(Device& dev, std::vector<float> x, int64_t rows, std::vector<float> g, std::vector<float> b,
                   std::vector<double> want, double atol) {
  const int64_t cols = static_cast<int64_t>(g.size());
  const Layout lx{rows, cols}, lv{cols};
  auto out = run(node("LAYER_NORM", lx, {OpRef::leaf(lx), OpRef::leaf(lv), OpRef::leaf(lv)}, {{"eps", 1e-5}, {"axis", -1}}),
                 {upload(dev, x), upload(dev, g), upload(dev, b)}, dev);
  return close_to(download(out[0]), want, atol, "y");
}

std::string ln_bwd(Device& dev, std::vector<float> dy, std::vector<float> x, int64_t rows, std::vector<float> g,
                   const std::vector<double>* dx, const std::vector<double>* dg, const std::vector<double>* db, double atol) {
  const int64_t cols = static_cast<int64_t>(g.size());
  const Layout lx{rows, cols}, lv{cols};
  auto out = run(node("LAYER_NORM_GRAD", lx, {OpRef::leaf(lx), OpRef::leaf(lx), OpRef::leaf(lv)}, {{"eps", 1e-5}, {"axis", -1}}),
                 {upload(dev, dy), upload(dev, x), upload(dev, g)}, dev);
  if (out.size() != 3) return "expected three outputs";
  std::string why;
  if (dx && why.empty()) why = close_to(download(out[0]), *dx, atol, "dx");
  if (dg && why.empty()) why = close_to(download(out[1]), *dg, atol, "dgamma");
  if (db && why.empty()) why = close_to(download(out[2]), *db, atol, "dbeta");
  return why;
}

// ---- cross-entropy ---------------------------------------------------------------------------------

std::string ce_loss(Device& dev, const std::vector<float>& logits, const Layout& la, const std::vector<float>& labels,
                    const Layout& lb, double want, double atol) {
  auto bl = upload(dev, logits).view(la);
  auto by = upload(dev, labels).view(lb);
  auto out = run(node("CROSS_ENTROPY", Layout{1}, {OpRef::leaf(la), OpRef::leaf(lb)}), {bl, by}, dev);
  return close_to(download(out[0]), {want}, atol, "loss");
}

// ---- small exact integers ------------------------------------------------------------------------

std::vector<float> ints(int64_t n, int seed, int lo, int hi) {
  std::vector<float> v(static_cast<size_t>(n));
  uint32_t s = 12345u + 977u * static_cast<uint32_t>(seed);
  for (auto& e : v) {
    s = s * 1664525u + 1013904223u;
    e = static_cast<float>(lo + static_cast<int>((s >> 8) % static_cast<uint32_t>(hi - lo + 1)));
  }
  return v;
}

}  // namespace

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "";
  if (mode == "rules") {
    for (const Rule& r : scheduler_rules()) std::printf("%s %s\n", r.op_type, r.exec_name);
    return 0;
  }
  if (mode != "run") {
    std::fprintf(stderr, "usage: %s rules | run\n", argv[0]);
    return 2;
  }

  std::unique_ptr<Device> holder;
  try {
    holder = std::make_unique<Device>(0);
  } catch (const Error& e) {
    std::fprintf(stderr, "selftest: %s\n", e.what());
    return 3;
  }
  Device& dev = *holder;

  // tests/test_nn.mojo:283-324
  run_case("layer_norm_fwd golden gamma/beta", [&] {
    return ln_fwd(dev, {1, 2, 3, 4}, 1, {1, 2, 1, 2}, {0.1f, 0.2f, 0.1f, 0.2f}, {-1.241641, -0.694427, 0.547214, 2.883282}, 1e-4);
  });
  run_case("layer_norm_fwd golden two rows", [&] {
    return ln_fwd(dev, {1, 2, 3, 4, -1, -2, -3, -4}, 2, {1, 1, 1, 1}, {0, 0, 0, 0},
                  {-1.341641, -0.447214, 0.447214, 1.341641, 1.341641, 0.447214, -0.447214, -1.341641}, 1e-4);
  });
  run_case("layer_norm_fwd constant row gives beta", [&] {
    return ln_fwd(dev, {3, 3, 3, 3}, 1, {1, 1, 1, 1}, {0.5f, 0.5f, 0.5f, 0.5f}, {0.5, 0.5, 0.5, 0.5}, 1e-4);
  });
  // tests/test_grad.mojo:776-856
  run_case("layer_norm_bwd golden", [&] {
    const std::vector<double> dx{0.0, 0.089443, -0.178886, 0.089443}, dg{-0.134164, -0.089443, 0.134164, 0.536656},
        db{0.1, 0.2, 0.3, 0.4};
    return ln_bwd(dev, {0.1f, 0.2f, 0.3f, 0.4f}, {1, 2, 3, 4}, 1, {1, 2, 1, 2}, &dx, &dg, &db, 2e-4);
  });
  run_case("layer_norm_bwd two identical rows double dbeta", [&] {
    const std::vector<double> db{0.2, 0.4, 0.6, 0.8};
    return ln_bwd(dev, {0.1f, 0.2f, 0.3f, 0.4f, 0.1f, 0.2f, 0.3f, 0.4f}, {1, 2, 3, 4, 1, 2, 3, 4}, 2, {1, 1, 1, 1}, nullptr,
                  nullptr, &db, 1e-5);
  });
  run_case("layer_norm_bwd uniform dy gives zero dx", [&] {
    const std::vector<double> dx{0, 0, 0, 0};
    return ln_bwd(dev, {1, 1, 1, 1}, {1, 2, 3, 4}, 1, {1, 1, 1, 1}, &dx, nullptr, nullptr, 1e-5);
  });

  // tests/test_ops.mojo:155-175
  run_case("cross_entropy zeros (4,10) one-hot = ln 10", [&] {
    std::vector<float> labels(40, 0.f);
    for (int i = 0; i < 4; ++i) labels[i * 10 + i] = 1.f;
    return ce_loss(dev, std::vector<float>(40, 0.f), Layout{4, 10}, labels, Layout{4, 10}, 2.302585, 1e-3);
  });
  run_case("cross_entropy soft labels = ln 4", [&] {
    return ce_loss(dev, std::vector<float>(8, 0.f), Layout{2, 4}, std::vector<float>(8, 0.25f), Layout{2, 4}, 1.386294, 1e-3);
  });
  run_case("cross_entropy certain prediction = 0", [&] {
    return ce_loss(dev, {100, 0, 0, 0, 100, 0}, Layout{2, 3}, {1, 0, 0, 0, 1, 0}, Layout{2, 3}, 0.0, 1e-3);
  });
  // tests/test_non_contiguous.mojo:275-299: the strided route (every other row; transposed labels)
  run_case("cross_entropy strided logits = ln 2", [&] {
    const Layout sl = Layout{4, 2}.slice_axis(0, 0, 4, 2);
    if (sl.is_contiguous()) return std::string("slice should not be contiguous");
    return ce_loss(dev, {0, 0, 100, 0, 0, 0, 0, 0}, sl, {0.5f, 0.5f, 0.5f, 0.5f}, Layout{2, 2}, 0.693147, 1e-3);
  });
  run_case("cross_entropy transposed labels = ln 2", [&] {
    return ce_loss(dev, {0, 0, 0, 0}, Layout{2, 2}, {1, 0, 0, 1}, Layout{2, 2}.transpose(), 0.693147, 1e-3);
  });
  // tests/test_non_contiguous.mojo:302-310: logits = a^T, labels = I; expected is d/da
  run_case("cross_entropy_grad golden on a transposed view", [&] {
    const Layout la = Layout{2, 2}.transpose(), lb{2, 2};
    auto out = run(node("CROSS_ENTROPY_GRAD", la.as_contiguous(), {OpRef::leaf(la), OpRef::leaf(lb), OpRef::leaf(Layout{1})}),
                   {upload(dev, {1, 2, 3, 4}).view(la), upload(dev, {1, 0, 0, 1}), upload(dev, {1.0f})}, dev);
    const auto d = download(out[0]);  // dlogits (2,2); d/da is its transpose
    return close_to({d[0], d[2], d[1], d[3]}, {-0.440398, 0.059601, 0.440398, -0.059601}, 1e-3, "grad");
  });

  // Attention closed forms, fp32 tensors (tests/test_ops.mojo:903-946, tests/test_grad.mojo:1001-1023)
  run_case("flash_attn closed forms", [&] {
    const int64_t B = 1, S = 32, H = 1, D = 8;
    const Layout bshd{B, S, H, D}, bhsd{B, H, S, D};
    const auto v = ints(B * S * H * D, 1, -3, 3);
    const std::vector<float> zeros(static_cast<size_t>(B * S * H * D), 0.f), ones(zeros.size(), 1.f);
    auto bq = upload(dev, zeros), bk = upload(dev, zeros), bv = upload(dev, v), mask = upload(dev, {0.f});
    const std::map<std::string, double> causal{{"scale", 1.0 / std::sqrt(8.0)}, {"is_causal", 1}, {"has_bias", 0}};
    auto fwd = run(node("FLASH_ATTN", bhsd, {OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(Layout{1})}, causal),
                   {bq, bk, bv, mask}, dev);
    const auto o = download(fwd[0]);
    // Q = K = 0, causal: row i of O is the mean of V[0..i]; row 0 is V[0]
    for (int64_t d = 0; d < D; ++d)
      if (std::fabs(o[d] - v[d]) > 1e-6) return std::string("causal row 0 is not V[0]");
    std::vector<double> want(static_cast<size_t>(S * D), 0.0);
    for (int64_t d = 0; d < D; ++d) {
      double run_sum = 0;
      for (int64_t i = 0; i < S; ++i) {
        run_sum += v[i * D + d];
        want[i * D + d] = run_sum / (i + 1);
      }
    }
    std::string why = close_to(o, want, 1e-5, "O");
    if (!why.empty()) return why;
    const auto lse = download(fwd[1]);
    for (int64_t i = 0; i < S; ++i)
      if (std::fabs(lse[i] - std::log(static_cast<double>(i + 1))) > 1e-5) return std::string("lse is not ln(i+1)");
    // loss = sum(O): dV[j] = sum_{i>=j} 1/(i+1) in every column; dQ = dK = 0
    auto bwd = run(node("FLASH_ATTN_GRAD", bshd,
                        {OpRef::leaf(bhsd), OpRef::leaf(bhsd), OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(bshd),
                         OpRef::leaf(Layout{1}), OpRef::leaf(Layout{B, H, S})},
                        {{"scale", 1.0 / std::sqrt(8.0)}, {"is_causal", 1}}),  // has_bias defaults to not causal
                   {upload(dev, ones), fwd[0], bq, bk, bv, mask, fwd[1]}, dev);
    std::vector<double> dv(static_cast<size_t>(S * D));
    for (int64_t j = 0; j < S; ++j) {
      double tail = 0;
      for (int64_t i = j; i < S; ++i) tail += 1.0 / (i + 1);
      for (int64_t d = 0; d < D; ++d) dv[j * D + d] = tail;
    }
    why = close_to(download(bwd[2]), dv, 1e-5, "dV");
    if (!why.empty()) return why;
    // With Q = K = 0 and dP rows that are affine in V: dS = P (dP - delta) need not vanish, but
    // dQ = dS K = 0 because K = 0; dK = dS^T Q = 0 because Q = 0.
    const std::vector<double> zero(static_cast<size_t>(S * D), 0.0);
    why = close_to(download(bwd[0]), zero, 1e-6, "dQ");
    if (!why.empty()) return why;
    return close_to(download(bwd[1]), zero, 1e-6, "dK");
  });

  // Linear layer forward and gradients through the reference's call patterns (mograd/grad.mojo:180-187):
  // Y = X W^T + b (MATMUL_BIAS_BT); dX = dY W as MATMUL_BT with B = W^T view (strides (1, K));
  // dW^T = X^T dY as MATMUL with A = X^T view; db = SUM{axis 0}.  Small integers: exact in fp32.
  run_case("linear forward and gradients, exact integers", [&] {
    const int64_t M = 37, N = 29, K = 53;
    const auto x = ints(M * K, 2, -4, 4), w = ints(N * K, 3, -4, 4), b = ints(N, 4, -9, 9), dy = ints(M * N, 5, -4, 4);
    const Layout lx{M, K}, lw{N, K}, lb{N}, ly{M, N};
    auto bx = upload(dev, x), bw = upload(dev, w), bb = upload(dev, b), bdy = upload(dev, dy);
    auto y = run(node("MATMUL_BIAS_BT", ly, {OpRef::leaf(lx), OpRef::leaf(lw), OpRef::leaf(lb)}), {bx, bw, bb}, dev);
    std::vector<double> want(static_cast<size_t>(M * N));
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < N; ++n) {
        double s = b[n];
        for (int64_t k = 0; k < K; ++k) s += static_cast<double>(x[m * K + k]) * w[n * K + k];
        want[m * N + n] = s;
      }
    std::string why = close_to(download(y[0]), want, 0.0, "Y");
    if (!why.empty()) return why;
    // dX (M,K) = dY (M,N) . W (N,K): A = dY, B^T = W, i.e. B = W^T view of shape (K,N)
    const Layout wt = lw.transpose();
    auto dx = run(node("MATMUL_BT", lx, {OpRef::leaf(ly), OpRef::leaf(wt)}), {bdy, bw.view(wt)}, dev);
    want.assign(static_cast<size_t>(M * K), 0.0);
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k) {
        double s = 0;
        for (int64_t n = 0; n < N; ++n) s += static_cast<double>(dy[m * N + n]) * w[n * K + k];
        want[m * K + k] = s;
      }
    why = close_to(download(dx[0]), want, 0.0, "dX");
    if (!why.empty()) return why;
    // dW^T (K,N) = X^T (K,M) . dY (M,N)
    const Layout xt = lx.transpose();
    auto dwt = run(node("MATMUL", Layout{K, N}, {OpRef::leaf(xt), OpRef::leaf(ly)}), {bx.view(xt), bdy}, dev);
    want.assign(static_cast<size_t>(K * N), 0.0);
    for (int64_t k = 0; k < K; ++k)
      for (int64_t n = 0; n < N; ++n) {
        double s = 0;
        for (int64_t m = 0; m < M; ++m) s += static_cast<double>(x[m * K + k]) * dy[m * N + n];
        want[k * N + n] = s;
      }
    why = close_to(download(dwt[0]), want, 0.0, "dW^T");
    if (!why.empty()) return why;
    auto db = run(node("SUM", lb, {OpRef::leaf(ly)}, {{"axis", 0}}), {bdy}, dev);
    want.assign(static_cast<size_t>(N), 0.0);
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < N; ++n) want[n] += dy[m * N + n];
    return close_to(download(db[0]), want, 0.0, "db");
  });

  // The gradient rule the reference lacks: MATMUL_BIAS_BT -> one LINEAR_GRAD node whose three
  // outputs are dX, dW (in W's layout) and db.  Same integers as above: exact in fp32.
  run_case("linear_grad rule: MATMUL_BIAS_BT -> LINEAR_GRAD, exact integers", [&] {
    const int64_t M = 37, N = 29, K = 53;
    const auto x = ints(M * K, 2, -4, 4), w = ints(N * K, 3, -4, 4), dy = ints(M * N, 5, -4, 4);
    const Layout lx{M, K}, lw{N, K}, lb{N}, ly{M, N};
    const OpRef fwd = node("MATMUL_BIAS_BT", ly, {OpRef::leaf(lx), OpRef::leaf(lw), OpRef::leaf(lb)});
    const OpRef bwd = linear_grad(fwd, OpRef::leaf(ly));
    if (bwd.op_type != "LINEAR_GRAD" || bwd.srcs.size() != 3 || bwd.attr("has_bias") != 1) return std::string("wrong node");
    auto out = run(bwd, {upload(dev, dy), upload(dev, x), upload(dev, w)}, dev);
    if (out.size() != 3) return std::string("expected three outputs");
    std::vector<double> want(static_cast<size_t>(M * K), 0.0);
    for (int64_t m = 0; m < M; ++m)
      for (int64_t k = 0; k < K; ++k)
        for (int64_t n = 0; n < N; ++n) want[m * K + k] += static_cast<double>(dy[m * N + n]) * w[n * K + k];
    std::string why = close_to(download(out[0]), want, 0.0, "dX");
    if (!why.empty()) return why;
    want.assign(static_cast<size_t>(N * K), 0.0);
    for (int64_t n = 0; n < N; ++n)
      for (int64_t k = 0; k < K; ++k)
        for (int64_t m = 0; m < M; ++m) want[n * K + k] += static_cast<double>(dy[m * N + n]) * x[m * K + k];
    why = close_to(download(out[1]), want, 0.0, "dW");
    if (!why.empty()) return why;
    want.assign(static_cast<size_t>(N), 0.0);
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < N; ++n) want[n] += dy[m * N + n];
    why = close_to(download(out[2]), want, 0.0, "db");
    if (!why.empty()) return why;
    // MATMUL_BT (no bias): two outputs
    const OpRef bwd2 = linear_grad(node("MATMUL_BT", ly, {OpRef::leaf(lx), OpRef::leaf(lw)}), OpRef::leaf(ly));
    return std::string(run(bwd2, {upload(dev, dy), upload(dev, x), upload(dev, w)}, dev).size() == 2 ? "" : "expected two outputs");
  });
  // LAYER_NORM as a multi-output node whose statistics feed the backward: the golden vectors of
  // tests/test_nn.mojo:283-324 and tests/test_grad.mojo:776-856 through the new pair.
  run_case("layer_norm_stats pair reproduces the goldens", [&] {
    const Layout lx{1, 4}, lv{4}, lr{1};
    const OpRef fwd = node("LAYER_NORM_STATS", lx, {OpRef::leaf(lx), OpRef::leaf(lv), OpRef::leaf(lv)}, {{"eps", 1e-5}});
    auto bx = upload(dev, {1, 2, 3, 4}), bg = upload(dev, {1, 2, 1, 2});
    auto out = run(fwd, {bx, bg, upload(dev, {0.1f, 0.2f, 0.1f, 0.2f})}, dev);
    if (out.size() != 3) return std::string("expected y, mean, rstd");
    std::string why = close_to(download(out[0]), {-1.241641, -0.694427, 0.547214, 2.883282}, 1e-4, "y");
    if (why.empty()) why = close_to(download(out[1]), {2.5}, 1e-6, "mean");
    if (why.empty()) why = close_to(download(out[2]), {1.0 / std::sqrt(1.25 + 1e-5)}, 1e-5, "rstd");
    if (!why.empty()) return why;
    const OpRef bwd = layer_norm_stats_grad(fwd, OpRef::leaf(lx), OpRef::leaf(lr), OpRef::leaf(lr));
    auto g = run(bwd, {upload(dev, {0.1f, 0.2f, 0.3f, 0.4f}), bx, bg, out[1], out[2]}, dev);
    why = close_to(download(g[0]), {0.0, 0.089443, -0.178886, 0.089443}, 2e-4, "dx");
    if (why.empty()) why = close_to(download(g[1]), {-0.134164, -0.089443, 0.134164, 0.536656}, 2e-4, "dgamma");
    if (why.empty()) why = close_to(download(g[2]), {0.1, 0.2, 0.3, 0.4}, 1e-6, "dbeta");
    return why;
  });
  // Class-id labels: the goldens of tests/test_ops.mojo:155-175 with ids in place of one-hot rows,
  // and the gradient golden of tests/test_non_contiguous.mojo:302-310 on a contiguous copy.
  run_case("cross_entropy_ids and its gradient rule", [&] {
    const Layout la{4, 10}, li{4};
    const int32_t host_ids[4] = {0, 1, 2, 3};
    AnyBuffer ids = AnyBuffer::from_host(dev, host_ids, 4, int32);
    OpRef fwd = node("CROSS_ENTROPY_IDS", Layout{1}, {OpRef::leaf(la), OpRef::leaf(li, int32)});
    auto loss = run(fwd, {upload(dev, std::vector<float>(40, 0.f)), ids}, dev);
    std::string why = close_to(download(loss[0]), {2.302585}, 1e-3, "loss");
    if (!why.empty()) return why;
    // logits [[1,3],[2,4]], labels (0,1): d/dlogits = (softmax - onehot) / 2
    const Layout l2{2, 2}, i2{2};
    const int32_t host_ids2[2] = {0, 1};
    AnyBuffer ids2 = AnyBuffer::from_host(dev, host_ids2, 2, int32);
    const OpRef f2 = node("CROSS_ENTROPY_IDS", Layout{1}, {OpRef::leaf(l2), OpRef::leaf(i2, int32)});
    const OpRef g2 = cross_entropy_ids_grad(f2, OpRef::leaf(Layout{1}));
    if (g2.op_type != "CROSS_ENTROPY_IDS_GRAD") return std::string("wrong node");
    auto d = run(g2, {upload(dev, {1, 3, 2, 4}), ids2, upload(dev, {1.0f})}, dev);
    return close_to(download(d[0]), {-0.440398, 0.440398, 0.059601, -0.059601}, 1e-3, "grad");
  });

  run_case("relu_grad is a bit-exact select", [&] {
    const auto out = ints(1000, 6, -2, 2), up = ints(1000, 7, -9, 9);
    const Layout l{1000};
    auto g = run(node("RELU_GRAD", l, {OpRef::leaf(l), OpRef::leaf(l)}), {upload(dev, out), upload(dev, up)}, dev);
    std::vector<double> want(1000);
    for (int i = 0; i < 1000; ++i) want[i] = out[i] > 0 ? up[i] : 0.0;
    return close_to(download(g[0]), want, 0.0, "dx");
  });

  run_case("elementwise maps and softmax read views in place", [&]() -> std::string {
    // (6, 8) values; a bias row broadcast over the rows; the transpose of the values
    const int64_t R = 6, C = 8;
    const auto a = ints(R * C, 8, -5, 5), bias = ints(C, 9, -3, 3);
    const Layout la{R, C}, lbias({R, C}, {0, 1}), lt({C, R}, {1, C});
    auto sum = run(node("ADD", la, {OpRef::leaf(la), OpRef::leaf(lbias)}), {upload(dev, a), upload(dev, bias).view(lbias)}, dev);
    std::vector<double> want(R * C);
    for (int64_t i = 0; i < R; ++i)
      for (int64_t j = 0; j < C; ++j) want[i * C + j] = a[i * C + j] + bias[j];
    std::string why = close_to(download(sum[0]), want, 0.0, "a + bias row");
    if (!why.empty()) return why;
    auto rt = run(node("RELU", Layout{C, R}, {OpRef::leaf(lt)}), {upload(dev, a).view(lt)}, dev);
    for (int64_t j = 0; j < C; ++j)
      for (int64_t i = 0; i < R; ++i) want[j * R + i] = std::max(a[i * C + j], 0.0f);
    why = close_to(download(rt[0]), want, 0.0, "relu of the transpose");
    if (!why.empty()) return why;
    auto gt = run(node("RELU_GRAD", Layout{C, R}, {OpRef::leaf(lt), OpRef::leaf(Layout{C, R})}),
                  {upload(dev, a).view(lt), upload(dev, ints(R * C, 10, -9, 9))}, dev);
    const auto up = ints(R * C, 10, -9, 9);
    for (int64_t j = 0; j < C; ++j)
      for (int64_t i = 0; i < R; ++i) want[j * R + i] = a[i * C + j] > 0 ? up[j * R + i] : 0.0;
    why = close_to(download(gt[0]), want, 0.0, "relu_grad with a transposed output");
    if (!why.empty()) return why;
    // softmax down the columns of zeros: every entry 1 / R
    auto sm = run(node("SOFTMAX", Layout{C, R}, {OpRef::leaf(lt)}), {upload(dev, std::vector<float>(R * C, 0.f)).view(lt)}, dev);
    return close_to(download(sm[0]), std::vector<double>(R * C, 1.0 / R), 1e-6, "softmax of a transposed view");
  });

  // Error conditions of the reference, with its messages
  run_case("matmul rejects non-collapsible batch dims", [&]() -> std::string {
    // transpose(1, 2) of a rank-4 tensor: batch dims no longer fold into one stride (kernels/__init__.mojo:633-634)
    const Layout a = Layout{2, 3, 4, 5}.transpose(0, 1), b{5, 6};
    try {
      run(node("MATMUL", Layout{3, 2, 4, 6}, {OpRef::leaf(a), OpRef::leaf(b)}), {upload(dev, std::vector<float>(120)), upload(dev, std::vector<float>(30))}, dev);
    } catch (const Error& e) {
      return std::strstr(e.what(), "non-collapsible batch dims") ? "" : std::string("wrong message: ") + e.what();
    }
    return "no error raised";
  });
  run_case("flash_attn rejects causal with bias", [&]() -> std::string {
    // kernels/__init__.mojo:868-873
    const Layout bshd{1, 4, 1, 8}, bhsd{1, 1, 4, 8};
    auto z = upload(dev, std::vector<float>(32, 0.f));
    try {
      run(node("FLASH_ATTN", bhsd, {OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(Layout{1, 1, 4, 4})},
               {{"scale", 1.0}, {"is_causal", 1}}),  // has_bias defaults to true in the forward dispatch
          {z, z, z, upload(dev, std::vector<float>(16, 0.f))}, dev);
    } catch (const Error& e) {
      return e.code == MG_ERR_INVALID ? "" : std::string("wrong status: ") + e.what();
    }
    return "no error raised";
  });
  run_case("unknown op has no rule", [&]() -> std::string {
    try {
      run(node("CONV2D", Layout{1}, {}), {}, dev);
    } catch (const Error& e) {
      return e.code == MG_ERR_UNSUPPORTED ? "" : "wrong status";
    }
    return "no error raised";
  });

  // The fused nodes that the rewrite rules create, against the nodes they replace, on small
  // integers (every sum exact in fp32, so equality is exact whatever the order): a block's
  // residual product, its ReLU product, the ReLU gradient folded into LINEAR_GRAD, LayerNorm's
  // gradient added to the skip connection's, and the same gradients with their second-stage sums
  // deferred to one launch.
  run_case("rewrites: fused nodes equal the nodes they replace", [&]() -> std::string {
    const int64_t M = 64, N = 24, K = 40;
    const Layout lx{M, K}, lw{N, K}, ly{M, N}, lb{N};
    const auto x = ints(M * K, 21, -3, 3), w = ints(N * K, 22, -2, 2), b = ints(N, 23, -4, 4), r = ints(M * N, 24, -9, 9);
    Buffers in = {upload(dev, x), upload(dev, w), upload(dev, b), upload(dev, r)};
    const OpRef nx = OpRef::leaf(lx), nw = OpRef::leaf(lw), nb = OpRef::leaf(lb), nr = OpRef::leaf(ly);
    // ADD(MATMUL_BT, r) -> MATMUL_BT_ADD
    const OpRef mm = node("MATMUL_BT", ly, {nx, nw});
    const auto fused_add = fuse_matmul_add(node("ADD", ly, {nr, mm}));
    if (!fused_add || fused_add->op_type != "MATMUL_BT_ADD") return "ADD(r, MATMUL_BT) was not rewritten";
    auto y0 = run(mm, {in[0], in[1]}, dev);
    auto y1 = run(node("ADD", ly, {nr, mm}), {in[3], y0[0]}, dev);
    auto y2 = run(*fused_add, {in[0], in[1], in[3]}, dev);
    if (download(y1[0]) != download(y2[0])) return "MATMUL_BT_ADD differs from MATMUL_BT + ADD";
    // RELU(MATMUL_BIAS_BT) -> MATMUL_BIAS_RELU_BT
    const OpRef mb = node("MATMUL_BIAS_BT", ly, {nx, nw, nb});
    const auto fused_relu = fuse_matmul_bias_relu(node("RELU", ly, {mb}));
    if (!fused_relu || fused_relu->op_type != "MATMUL_BIAS_RELU_BT") return "RELU(MATMUL_BIAS_BT) was not rewritten";
    auto a0 = run(mb, {in[0], in[1], in[2]}, dev);
    auto a1 = run(node("RELU", ly, {mb}), {a0[0]}, dev);
    auto a2 = run(*fused_relu, {in[0], in[1], in[2]}, dev);
    if (download(a1[0]) != download(a2[0])) return "MATMUL_BIAS_RELU_BT differs from MATMUL_BIAS_BT + RELU";
    // RELU_GRAD(y, LINEAR_GRAD[0]) -> LINEAR_GRAD{relu_mask}: here x plays the ReLU's output
    std::vector<float> xr = x;
    for (auto& v : xr) v = v > 0 ? v : 0;
    AnyBuffer bx = upload(dev, xr), bdy = upload(dev, r);
    const OpRef lin = linear_grad(node("MATMUL_BT", ly, {nx, nw}), nr);
    const OpRef sel = gettuple(lin, 0, lx, float32);
    const auto masked = fuse_relu_grad_into_linear_grad(node("RELU_GRAD", lx, {nx, sel}), true);
    if (!masked || masked->src(0).attr("relu_mask") != 1) return "RELU_GRAD(y, LINEAR_GRAD[0]) was not rewritten";
    auto g0 = run(lin, {bdy, bx, in[1]}, dev);
    auto g1 = run(node("RELU_GRAD", lx, {nx, sel}), {bx, g0[0]}, dev);
    auto g2 = run(masked->src(0), {bdy, bx, in[1]}, dev);
    if (download(g1[0]) != download(g2[0])) return "LINEAR_GRAD{relu_mask} differs from LINEAR_GRAD + RELU_GRAD";
    if (download(g0[1]) != download(g2[1])) return "dW changed under relu_mask";
    // ADD(p, LINEAR_GRAD[0]) -> LINEAR_GRAD{accumulate}
    const auto accum = fuse_add_into_linear_grad(node("ADD", lx, {nx, sel}));
    if (!accum || accum->src(0).srcs.size() != 4) return "ADD(p, LINEAR_GRAD[0]) was not rewritten";
    auto p1 = run(node("ADD", lx, {nx, sel}), {in[0], g0[0]}, dev);
    auto p2 = run(accum->src(0), {bdy, bx, in[1], in[0]}, dev);
    if (download(p1[0]) != download(p2[0])) return "LINEAR_GRAD{accumulate} differs from LINEAR_GRAD + ADD";
    // the same LINEAR_GRAD with its second-stage sums deferred
    {
      DeferredSums sums(dev);
      auto d2 = run(masked->src(0), {bdy, bx, in[1]}, dev);
      sums.finish();
      if (download(d2[0]) != download(g2[0]) || download(d2[1]) != download(g2[1])) return "deferred LINEAR_GRAD differs";
    }
    return "";
  });
  run_case("rewrites: LayerNorm gradient added to the skip connection's", [&]() -> std::string {
    const int64_t rows = 48, cols = 32;
    const Layout lx{rows, cols}, lv{cols}, lr{rows};
    const auto x = ints(rows * cols, 31, -5, 5), dy = ints(rows * cols, 32, -3, 3), res = ints(rows * cols, 33, -7, 7);
    std::vector<float> g(cols, 1.f), b(cols, 0.f);
    for (int64_t c = 0; c < cols; ++c) g[c] = 0.5f + 0.125f * static_cast<float>(c % 8);
    const OpRef fwd = node("LAYER_NORM_STATS", lx, {OpRef::leaf(lx), OpRef::leaf(lv), OpRef::leaf(lv)}, {{"eps", 1e-5}});
    AnyBuffer bx = upload(dev, x), bg = upload(dev, g), bdy = upload(dev, dy), bres = upload(dev, res);
    auto f = run(fwd, {bx, bg, upload(dev, b)}, dev);
    const OpRef bwd = layer_norm_stats_grad(fwd, OpRef::leaf(lx), OpRef::leaf(lr), OpRef::leaf(lr));
    const OpRef sel = gettuple(bwd, 0, lx, float32);
    const auto fused = fuse_add_into_layer_norm_grad(node("ADD", lx, {OpRef::leaf(lx), sel}));
    if (!fused || fused->src(0).op_type != "LAYER_NORM_STATS_GRAD_ADD") return "ADD(r, LAYER_NORM_STATS_GRAD[0]) was not rewritten";
    auto g0 = run(bwd, {bdy, bx, bg, f[1], f[2]}, dev);
    auto g1 = run(node("ADD", lx, {OpRef::leaf(lx), sel}), {bres, g0[0]}, dev);
    auto g2 = run(fused->src(0), {bdy, bx, bg, f[1], f[2], bres}, dev);
    if (download(g1[0]) != download(g2[0])) return "dx differs from LAYER_NORM_STATS_GRAD + ADD";
    if (download(g0[1]) != download(g2[1]) || download(g0[2]) != download(g2[2])) return "dgamma / dbeta changed";
    DeferredSums sums(dev);
    auto g3 = run(fused->src(0), {bdy, bx, bg, f[1], f[2], bres}, dev);
    sums.finish();
    if (download(g3[0]) != download(g2[0]) || download(g3[1]) != download(g2[1]) || download(g3[2]) != download(g2[2]))
      return "deferred sums differ";
    return "";
  });
  run_case("rewrites: a Linear layer's backward continued through the LayerNorm that feeds it", [&]() -> std::string {
    // fp32 tensors take the separate kernels inside the one entry: the same bits as the two nodes
    const int64_t rows = 48, cols = 32, N = 24;
    const Layout lh{rows, cols}, lv{cols}, lr{rows}, lw{N, cols}, ldy{rows, N};
    const auto h = ints(rows * cols, 51, -5, 5), dy = ints(rows * N, 52, -3, 3), w = ints(N * cols, 53, -2, 2),
               res = ints(rows * cols, 54, -7, 7);
    std::vector<float> g(cols, 1.f), b(cols, 0.f);
    for (int64_t c = 0; c < cols; ++c) g[c] = 0.5f + 0.125f * static_cast<float>(c % 8);
    const OpRef fwd = node("LAYER_NORM_STATS", lh, {OpRef::leaf(lh), OpRef::leaf(lv), OpRef::leaf(lv)}, {{"eps", 1e-5}});
    AnyBuffer bh = upload(dev, h), bg = upload(dev, g), bdy = upload(dev, dy), bw = upload(dev, w), bres = upload(dev, res);
    auto f = run(fwd, {bh, bg, upload(dev, b)}, dev);
    const OpRef x = gettuple(fwd, 0, lh, float32);
    const OpRef y = node("MATMUL_BIAS_BT", ldy, {x, OpRef::leaf(lw), OpRef::leaf(Layout{N})});
    const OpRef lin = linear_grad(y, OpRef::leaf(ldy));
    const OpRef ln = layer_norm_stats_grad(fwd, gettuple(lin, 0, lh, float32), OpRef::leaf(lr), OpRef::leaf(lr));
    const auto fused = fuse_linear_grad_into_layer_norm_grad(ln);
    if (!fused || fused->op_type != "LINEAR_LAYER_NORM_GRAD" || fused->srcs.size() != 7)
      return "LAYER_NORM_STATS_GRAD(LINEAR_GRAD[0], ..) was not rewritten";
    const auto accum = fuse_add_into_linear_layer_norm_grad(node("ADD", lh, {OpRef::leaf(lh), gettuple(*fused, 0, lh, float32)}));
    if (!accum || accum->src(0).srcs.size() != 8) return "ADD(r, LINEAR_LAYER_NORM_GRAD[0]) was not rewritten";
    auto l0 = run(lin, {bdy, f[0], bw}, dev);
    auto n0 = run(ln, {l0[0], bh, bg, f[1], f[2]}, dev);
    auto a0 = run(node("ADD", lh, {OpRef::leaf(lh), OpRef::leaf(lh)}), {bres, n0[0]}, dev);
    auto f1 = run(*fused, {bdy, f[0], bw, bh, bg, f[1], f[2]}, dev);
    auto f2 = run(accum->src(0), {bdy, f[0], bw, bh, bg, f[1], f[2], bres}, dev);
    if (download(f1[0]) != download(n0[0]) || download(f2[0]) != download(a0[0])) return "dh differs from the two nodes";
    if (download(f1[1]) != download(n0[1]) || download(f1[2]) != download(n0[2])) return "dgamma / dbeta differ";
    if (download(f1[3]) != download(l0[1]) || download(f1[4]) != download(l0[2])) return "dW / db differ";
    DeferredSums sums(dev);
    auto f3 = run(accum->src(0), {bdy, f[0], bw, bh, bg, f[1], f[2], bres}, dev);
    sums.finish();
    for (size_t i = 0; i < 5; ++i)
      if (download(f3[i]) != download(f2[i])) return "deferred sums differ";
    return "";
  });
  run_case("rewrites: attention output written (B, S, H, D)", [&]() -> std::string {
    const int64_t B = 1, S = 8, H = 2, D = 8;
    const Layout bshd{B, S, H, D}, bhsd{B, H, S, D};
    const auto q = ints(B * S * H * D, 41, -2, 2), k = ints(B * S * H * D, 42, -2, 2), v = ints(B * S * H * D, 43, -3, 3);
    Buffers in = {upload(dev, q), upload(dev, k), upload(dev, v), upload(dev, std::vector<float>(1, 0.f))};
    const OpRef attn = node("FLASH_ATTN", bhsd, {OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(bshd), OpRef::leaf(Layout{1})},
                            {{"scale", 0.25}, {"is_causal", 1}, {"has_bias", 0}});
    const OpRef o = gettuple(attn, 0, bhsd, float32);
    const OpRef tr = node("TRANSPOSE", bhsd.transpose(1, 2), {o}, {{"dim0", 1}, {"dim1", 2}});
    const OpRef copy = node("CONTIGUOUS", bshd, {tr});
    const auto fused = fuse_attention_output_layout(copy);
    if (!fused || fused->src(0).attr("layout") != kLayoutBshd) return "CONTIGUOUS(TRANSPOSE(FLASH_ATTN[0])) was not rewritten";
    auto a0 = run(attn, in, dev);
    auto t0 = run(tr, {a0[0]}, dev);
    auto c0 = run(copy, {t0[0]}, dev);
    auto a1 = run(fused->src(0), in, dev);
    if (download(c0[0]) != download(a1[0])) return "FLASH_ATTN{layout: bshd} differs from the copy";
    return "";
  });

  // Pool behaviour seen through AnyBuffer (tests/test_memory.mojo:18-60): a freed block of the
  // 1024-byte class serves the next request that rounds to the same class.
  run_case("pool reuses a size class", [&]() -> std::string {
    if (!dev.fn<decltype(&::mg_pool_enabled)>("mg_pool_enabled")()) return "";  // MOGRAD_POOL=0: nothing is cached
    void* first;
    {
      AnyBuffer a = AnyBuffer::create(float32, dev, 250);  // 1000 bytes -> class 1024
      first = a.data_ptr();
    }
    AnyBuffer b = AnyBuffer::create(float32, dev, 256);  // 1024 bytes -> same class
    const mg_pool_stats st = dev.memory_stats();
    if (st.hit_count < 1) return "no pool hit recorded";
    return b.data_ptr() == first ? "" : "a different block was handed out";
  });

  dev.synchronize();
  std::printf("%s: %d failed\n", g_failed ? "FAILED" : "OK", g_failed);
  return g_failed ? 1 : 0;
}
