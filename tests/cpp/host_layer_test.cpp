// C++ unit test of the host layer (no GPU needed): backend registration,
// function creation through the registry, Variable / NdArray / Half behaviour,
// the shape logic and the argument errors of every function class.  Built with
// -fsanitize=address,undefined by `make -C nnabla-ext-cuda_amd/csrc host_test`
// (the reference's counterpart is its gtest binary clibtest,
// src/nbla/cuda/test/test_nbla_cuda_utils.cpp:16-50).
#include <cmath>
#include <cstdio>
#include <functional>
#include <string>
#include <vector>

#include <nbla/function/batch_normalization.hpp>
#include <nbla/function/fused_batch_normalization.hpp>
#include <nbla/function/group_normalization.hpp>
#include <nbla/function/instance_normalization.hpp>
#include <nbla/function/layer_normalization.hpp>
#include <nbla/hip/init.hpp>
#include <nbla/variable.hpp>

using namespace nbla;

static int g_failed = 0, g_checks = 0;

#define EXPECT(cond)                                                       \
  do {                                                                     \
    ++g_checks;                                                            \
    if (!(cond)) {                                                         \
      ++g_failed;                                                          \
      std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
    }                                                                      \
  } while (0)

// Runs fn, expects an nbla::Exception whose text contains `needle`.
static void expect_throw(const std::function<void()> &fn, const char *needle, int line) {
  ++g_checks;
  try {
    fn();
  } catch (const Exception &e) {
    if (std::string(e.what()).find(needle) == std::string::npos) {
      ++g_failed;
      std::fprintf(stderr, "FAILED line %d: message lacks '%s': %s\n", line, needle, e.what());
    }
    return;
  }
  ++g_failed;
  std::fprintf(stderr, "FAILED line %d: no exception (expected '%s')\n", line, needle);
}
#define EXPECT_THROW(stmt, needle) expect_throw([&] { stmt; }, needle, __LINE__)

static void test_half() {
  const float values[] = {0.f, -0.f, 1.f, -2.5f, 65504.f, 6.1035156e-5f, 5.9604645e-8f, 1e-9f,
                          70000.f, 0.1f, 1.0009765625f, 1.00048828125f /* tie: to even */};
  for (float v : values) {
    const Half h(v);
    const float back = h;
    if (std::fabs(v) > 65504.f) {
      EXPECT(std::isinf(back));
    } else if (std::fabs(v) < 2.9802322e-8f) {
      EXPECT(back == 0.f);
    } else {
      EXPECT(std::fabs(back - v) <= std::fabs(v) * 9.765625e-4f + 6e-8f);
    }
  }
  EXPECT(static_cast<float>(Half(1.00048828125f)) == 1.0f);            // ties to even
  EXPECT(static_cast<float>(Half(1.00146484375f)) == 1.001953125f);    // ties to even, upward
  EXPECT(std::isnan(static_cast<float>(Half(std::nanf("")))));
  EXPECT(std::signbit(static_cast<float>(Half(-0.f))));
}

static void test_variable_and_arrays() {
  const Context cpu({"cpu:float"}, "CpuArray", "0");
  Variable v(Shape_t{2, 3, 4});
  EXPECT(v.size() == 24 && v.size(1) == 12 && v.size(3) == 1 && v.ndim() == 3);
  EXPECT((v.strides() == Shape_t{12, 4, 1}));
  float *d = v.cast_data_and_get_pointer<float>(cpu, true);
  for (int i = 0; i < 24; ++i) d[i] = 0.5f * static_cast<float>(i);
  const Half *h = v.get_data_pointer<Half>(cpu);            // dtype conversion on the host
  EXPECT(static_cast<float>(h[5]) == 2.5f);
  const float *f = v.get_data_pointer<float>(cpu);
  EXPECT(f[23] == 11.5f);
  // A reader's converted copy stays good until the next write: reading again
  // returns the same buffer without converting (a value planted in it
  // survives), and a write through cast() refreshes what the reader sees.
  const_cast<Half *>(h)[5] = Half(-7.f);
  const Half *h2 = v.get_data_pointer<Half>(cpu);
  EXPECT(h2 == h && static_cast<float>(h2[5]) == -7.f);
  EXPECT(v.get_data_pointer<float>(cpu)[5] == 2.5f);        // the head is untouched
  d = v.cast_data_and_get_pointer<float>(cpu, false);
  EXPECT(d[5] == 2.5f);
  d[5] = 9.f;
  EXPECT(static_cast<float>(v.get_data_pointer<Half>(cpu)[5]) == 9.f);
  v.grad()->fill(3.f);
  EXPECT(v.get_grad_pointer<float>(cpu)[7] == 3.f);
  v.grad()->zero();
  EXPECT(v.get_grad_pointer<float>(cpu)[7] == 0.f);
  EXPECT_THROW(v.reshape(Shape_t{5, 5}, false), "reshape");
  v.reshape(Shape_t{5, 5}, true);
  EXPECT(v.size() == 25);
  v.data()->array()->clear();
  for (int rep = 0; rep < 100; ++rep) {                     // churn for the leak checker
    Variable t(Shape_t{64, 64});
    t.data()->zero();
    (void)t.get_data_pointer<float>(cpu);
    t.data()->array()->clear();
  }
}

static Context hip_ctx(const char *tc) {
  return Context({std::string("hip:") + tc}, "HipCachedArray", "0");
}

static void test_registry() {
  init_hip();
  init_hip();                                               // idempotent
  const Context ctx = hip_ctx("float");
  EXPECT(create_BatchNormalization(ctx, vector<int>{1}, 0.9f, 1e-5f, true, false, false)->name() ==
         "BatchNormalizationHip");
  EXPECT(create_FusedBatchNormalization(ctx, vector<int>{1}, 0.9f, 1e-5f, true, string("relu"))->name() ==
         "FusedBatchNormalizationHip");
  EXPECT(create_LayerNormalization(hip_ctx("half"), vector<int>{0}, 1e-5f, false, false)->name() ==
         "LayerNormalizationHip");
  EXPECT(create_GroupNormalization(ctx, 2, 1, vector<int>{0}, 1e-5f, false, false)->name() ==
         "GroupNormalizationHip");
  EXPECT(create_InstanceNormalization(ctx, 1, vector<int>{0}, 1e-5f, false, false)->name() ==
         "InstanceNormalizationHip");
  // preference order: the first backend that has an implementation wins
  const Context mixed({"cudnn:float", "hip:half", "hip:float"}, "HipCachedArray", "0");
  EXPECT(create_LayerNormalization(mixed, vector<int>{0}, 1e-5f, true, true)->name() ==
         "LayerNormalizationHip");
  const Context cpu({"cpu:float"}, "CpuArray", "0");
  EXPECT_THROW(create_BatchNormalization(cpu, vector<int>{1}, 0.9f, 1e-5f, true, false, false),
               "No implementation");
}

// Shape logic and argument errors run before any device call.
static void test_setup_errors() {
  const Context ctx = hip_ctx("float");
  Variable x(Shape_t{4, 6, 5, 5}), y, p6(Shape_t{1, 6, 1, 1}), p5(Shape_t{1, 5, 1, 1});
  Variable m6(Shape_t{1, 6, 1, 1}), v6(Shape_t{1, 6, 1, 1});
  {
    auto f = create_BatchNormalization(ctx, vector<int>{1, 2}, 0.9f, 1e-5f, true, false, false);
    EXPECT_THROW(f->setup({&x, &p6, &p6, &m6, &v6}, {&y}), "more than one axis");
    auto g = create_BatchNormalization(ctx, vector<int>{1}, 0.9f, 1e-5f, true, false, false);
    EXPECT_THROW(g->setup({&x, &p5, &p6, &m6, &v6}, {&y}), "must have 6 elements");
    EXPECT_THROW(g->setup({&x, &p6, &m6, &v6}, {&y}), "expects 5 inputs");
    auto h = create_BatchNormalization(ctx, vector<int>{7}, 0.9f, 1e-5f, true, true, true);
    EXPECT_THROW(h->setup({&x, &m6, &v6}, {&y}), "out of range");
    EXPECT_THROW(g->forward({&x, &p6, &p6, &m6, &v6}, {&y}), "setup() was not called");
  }
  {
    auto f = create_FusedBatchNormalization(ctx, vector<int>{1}, 0.9f, 1e-5f, true, string("tanh"));
    EXPECT_THROW(f->setup({&x, &p6, &p6, &m6, &v6}, {&y}), "relu");
    auto g = create_FusedBatchNormalization(ctx, vector<int>{1}, 0.9f, 1e-5f, true, string("relu"));
    Variable z(Shape_t{4, 6, 5, 4});
    EXPECT_THROW(g->setup({&x, &p6, &p6, &m6, &v6, &z}, {&y}), "shape of x");
  }
  {
    auto f = create_LayerNormalization(ctx, vector<int>{9}, 1e-5f, true, true);
    EXPECT_THROW(f->setup({&x}, {&y}), "batch_axis out of range");
  }
  {
    auto f = create_GroupNormalization(ctx, 4, 1, vector<int>{0}, 1e-5f, true, true);
    EXPECT_THROW(f->setup({&x}, {&y}), "divisible");
    auto g = create_GroupNormalization(ctx, 1, 2, vector<int>{2}, 1e-5f, true, true);
    EXPECT_THROW(g->setup({&x}, {&y}), "batch_axis");   // batch axis equal to the channel axis
  }
  {
    auto f = create_InstanceNormalization(ctx, 1, vector<int>{0}, 1e-5f, false, false);
    Variable bad(Shape_t{1, 7, 1, 1});
    EXPECT_THROW(f->setup({&x, &bad, &p6}, {&y}), "beta/gamma");
  }
  {
    const Context wrong({"hip:float"}, "CpuArray", "0");
    auto f = create_LayerNormalization(wrong, vector<int>{0}, 1e-5f, true, true);
    EXPECT_THROW(f->setup({&x}, {&y}), "not allowed");
  }
}

int main() {
  init_hip(); // registers the array classes the Variables below live in
  test_half();
  test_variable_and_arrays();
  test_registry();
  test_setup_errors();
  std::printf("%d checks, %d failed\n", g_checks, g_failed);
  return g_failed ? 1 : 0;
}
