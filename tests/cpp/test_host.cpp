// C++ host-side tests.  Without arguments: CPU-only checks of the layout algebra (the reference's
// own unit tests, adrastea_models/src/tensor.rs:583-664, restated), the lowering rules
// (kernels.rs:821-890) and kernel selection.  With "gpu": one matmul through GpuKernels on the
// device (HIP runtime loaded with dlopen so that this file needs no HIP headers), checked against
// a host triple loop on integer-valued inputs.
#include <dlfcn.h>

#include <cstdio>
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../adrastea_amd/host/kernels.hpp"
#include "../../adrastea_amd/host/pickle.hpp"
#include "../../adrastea_amd/host/llama_loader.hpp"

using namespace adrastea;

static int failures = 0;
#define CHECK(c) do { if (!(c)) { printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #c); failures++; } } while (0)
template <typename F> static bool throws(F f) { try { f(); } catch (const std::exception&) { return true; } return false; }

static uint16_t f2h_small_int(int v) {  // exact fp16 of an integer |v| <= 2048
  if (v == 0) return 0;
  uint16_t sign = v < 0 ? 0x8000 : 0; unsigned a = v < 0 ? -v : v; int e = 0;
  while ((a >> (e + 1)) != 0) e++;
  return sign | (uint16_t)((e + 15) << 10) | (uint16_t)(((a << (10 - e)) & 0x3ff));
}
static int h2i(uint16_t h) {
  if ((h & 0x7fff) == 0) return 0;
  int e = ((h >> 10) & 31) - 15; int m = 0x400 | (h & 0x3ff); int v = e >= 10 ? m << (e - 10) : m >> (10 - e);
  return (h & 0x8000) ? -v : v;
}

static double h2d(uint16_t h) {  // any finite fp16 value
  const int e = (h >> 10) & 31, m = h & 0x3ff;
  const double mag = e ? (double)(0x400 | m) / 1024.0 * (e >= 15 ? (double)(1 << (e - 15)) : 1.0 / (double)(1 << (15 - e)))
                       : (double)m / 1024.0 / 16384.0;
  return (h & 0x8000) ? -mag : mag;
}

static void cpu_tests() {
  CHECK((TensorLayout::row_major({2, 3, 4}).strides == std::vector<size_t>{12, 4, 1}));
  CHECK((TensorLayout::column_major({3, 4}).strides == std::vector<size_t>{1, 4}));
  CHECK((TensorLayout::row_major({3, 3}).permute({1, 0}).strides == std::vector<size_t>{1, 3}));
  CHECK(TensorLayout::row_major({2, 3, 4}).largest_address() == 23);
  CHECK(throws([] { TensorLayout({2, 0}, {1, 1}); }));
  // shape_cast (tensor.rs:599-613) and its should_panic twin (:619-625)
  auto c = TensorLayout::row_major({4, 4}).shape_cast({-1, 8});
  CHECK((c.dims == std::vector<size_t>{2, 8}) && (c.strides == std::vector<size_t>{8, 1}));
  CHECK(throws([] { TensorLayout::row_major({256}).shape_cast({16, 1}); }));
  // skip_and_take (tensor.rs:627-664)
  auto r = TensorLayout::row_major({256}).shape_cast({16, 16});
  auto sk = r.skip({15, 0});
  CHECK(sk.first == 240 && sk.second.size(-2) == 1 && sk.second.size(-1) == 16);
  auto tk = r.skip({1, 0}).second.take({1, 16});
  CHECK(r.skip({1, 0}).first == 16 && tk.size(-2) == 1 && tk.size(-1) == 16);
  // LLaMA-7B attention views (llama.rs:534-554)
  const size_t S = 2048, H = 32, D = 128;
  auto base = TensorLayout::row_major({S, H * D});
  auto q = base.shape_cast({(long)S, (long)H, -1}).permute({1, 0, 2});
  auto k = base.shape_cast({(long)S, (long)H, -1}).permute({1, 2, 0});
  auto qk = TensorLayout::row_major({H, S, S});
  auto low = lower_matmul(qk, q, k, MatmulOptions::make().store(MatmulStore::Scale(0.0883883f)).mask(MatmulMask::Causal));
  CHECK(low.batches == 32 && low.m == 2048 && low.k == 128 && low.n == 2048);
  CHECK(low.sl[0] == 1 && low.sl[1] == 4096 && low.sl[2] == 128);
  CHECK(low.sr[0] == 4096 && low.sr[1] == 1 && low.sr[2] == 128);
  CHECK(low.so[0] == 1 && low.so[1] == 2048 && low.so[2] == 2048 * 2048);
  CHECK(low.store == 4 && low.load == 0 && low.mask == 1 && low.beta == 0.0f);
  // lowering rules
  auto out = TensorLayout::row_major({5, 7}), lhs = TensorLayout::row_major({5, 3});
  auto w = TensorLayout::row_major({7, 3}).permute({1, 0});
  auto l2 = lower_matmul(TensorLayout::row_major({4, 5, 7}), TensorLayout::row_major({4, 5, 3}), w, MatmulOptions::make());
  CHECK(l2.batches == 4 && l2.sr[2] == 0 && l2.sl[2] == 15);
  auto l3 = lower_matmul(out, lhs, w, MatmulOptions::make().load(MatmulLoad::Scale(0.5f)).store(MatmulStore::Scale(0.25f)));
  CHECK(l3.scale == 0.125f && l3.store == 4 && l3.load == 1);
  CHECK(lower_matmul(out, lhs, w, MatmulOptions::make().store(MatmulStore::BetaBias(1.0f, nullptr))).beta == 1.0f);
  CHECK(lower_matmul(out, lhs, w, MatmulOptions::make().store(MatmulStore::Add())).beta == 0.0f);
  CHECK(throws([&] { lower_matmul(TensorLayout::row_major({5, 8}), lhs, w, MatmulOptions::make()); }));
  CHECK(throws([&] { lower_matmul(out, TensorLayout::row_major({5, 4}), w, MatmulOptions::make()); }));
  // kernel selection through the library (host only)
  GpuKernels gk;
  auto big_o = TensorLayout::row_major({2048, 12288}), big_l = TensorLayout::row_major({2048, 4096});
  auto big_w = TensorLayout::row_major({12288, 4096}).permute({1, 0});
  CHECK(gk.plan(big_o, big_l, big_w, MatmulOptions::make()).rfind("gemm_nt_mfma", 0) == 0);
  CHECK(gk.plan(TensorLayout::row_major({10, 12}), TensorLayout::row_major({10, 7}), TensorLayout::row_major({7, 12}),
                MatmulOptions::make()) == "matmul_general");
  CHECK(throws([&] { gk.plan(out, lhs, w, MatmulOptions::make().store(MatmulStore::GeluBias(nullptr))); }));
}

static void gpu_test() {
  void* hip = dlopen("libamdhip64.so", RTLD_NOW);
  if (!hip) { printf("FAIL dlopen libamdhip64.so\n"); failures++; return; }
  auto hipMalloc = (int (*)(void**, size_t))dlsym(hip, "hipMalloc");
  auto hipMemcpy = (int (*)(void*, const void*, size_t, int))dlsym(hip, "hipMemcpy");
  auto hipDeviceSynchronize = (int (*)())dlsym(hip, "hipDeviceSynchronize");
  const int M = 70, K = 64, N = 96;
  std::vector<uint16_t> a(M * K), w(N * K), o(M * N, 0);
  unsigned s = 7;
  auto rnd = [&] { s = s * 1664525u + 1013904223u; return (int)((s >> 16) % 7) - 3; };
  for (auto& v : a) v = f2h_small_int(rnd());
  for (auto& v : w) v = f2h_small_int(rnd());
  uint16_t *da, *dw, *dout;
  CHECK(hipMalloc((void**)&da, a.size() * 2) == 0 && hipMalloc((void**)&dw, w.size() * 2) == 0 &&
        hipMalloc((void**)&dout, o.size() * 2) == 0);
  hipMemcpy(da, a.data(), a.size() * 2, 1); hipMemcpy(dw, w.data(), w.size() * 2, 1); hipMemcpy(dout, o.data(), o.size() * 2, 1);
  GpuKernels gk;
  MatmulTracer tr(gk);
  TensorView<f16> ov(dout, TensorLayout::row_major({(size_t)M, (size_t)N}));
  TensorView<const f16> lv(da, TensorLayout::row_major({(size_t)M, (size_t)K}));
  TensorView<const f16> wv(dw, TensorLayout::row_major({(size_t)N, (size_t)K}));
  for (int slow = 0; slow < 2; slow++) {
    if (slow) tr.matmul_f16_slow(ov, lv, wv.permute({1, 0}), MatmulOptions::make().mask(MatmulMask::Causal));
    else tr.matmul_f16(ov, lv, wv.permute({1, 0}), MatmulOptions::make().mask(MatmulMask::Causal));
    CHECK(hipDeviceSynchronize() == 0);
    hipMemcpy(o.data(), dout, o.size() * 2, 2);
    int bad = 0;
    for (int y = 0; y < M; y++)
      for (int x = 0; x < N; x++) {
        if (x > y) { bad += o[y * N + x] != 0xFC00; continue; }
        int ref = 0;
        for (int k = 0; k < K; k++) ref += h2i(a[y * K + k]) * h2i(w[x * K + k]);
        bad += h2i(o[y * N + x]) != ref;
      }
    CHECK(bad == 0);
  }
  CHECK(tr.shapes().size() == 1);
  // softmax_rows_inplace on the [M, N] result viewed as one head: rows of a causal product sum
  // to 1 and the masked entries become 0; error_stats of a tensor with itself is all zero
  tr.softmax_rows_inplace(ov, 1.0f);
  CHECK(hipDeviceSynchronize() == 0);
  hipMemcpy(o.data(), dout, o.size() * 2, 2);
  {
    int bad = 0;
    for (int y = 0; y < M; y++) {
      double sum = 0;
      for (int x = 0; x < N; x++) {
        const uint16_t h = o[y * N + x];
        if (x > y) { bad += h != 0; continue; }
        const int e = (h >> 10) & 31, m = h & 0x3ff;
        sum += e ? (double)(0x400 | m) / 1024.0 * (e >= 15 ? (double)(1 << (e - 15)) : 1.0 / (double)(1 << (15 - e)))
                 : (double)m / 1024.0 / 16384.0;
      }
      bad += !(sum > 0.99 && sum < 1.01);
    }
    CHECK(bad == 0);
  }
  {
    float* dstat;
    CHECK(hipMalloc((void**)&dstat, 12) == 0);
    float z[3] = {0, 0, 0};
    hipMemcpy(dstat, z, 12, 1);
    TensorView<float> sv(dstat, TensorLayout::row_major({3}));
    TensorView<const f16> cv(dout, TensorLayout::row_major({(size_t)M, (size_t)N}));
    tr.error_stats_f16(sv, cv, cv);
    CHECK(hipDeviceSynchronize() == 0);
    float st[3] = {1, 1, 1};
    hipMemcpy(st, dstat, 12, 2);
    CHECK(st[0] == 0.0f && st[1] == 0.0f && st[2] == 0.0f);
  }
  {
    // attention_f16 with zero queries: every score is equal, the output is the mean of the value
    // rows, exact here (64 keys, small-integer values); M x K reused as [1 head, M, K], K = d
    static_assert(K == 64 || K == 128, "head dimension of the fused kernel");
    const int NK = 64;
    std::vector<uint16_t> zq((size_t)M * K, 0), vv((size_t)NK * K), oo((size_t)M * K, 0);
    for (int x = 0; x < NK; x++)
      for (int c = 0; c < K; c++) vv[(size_t)x * K + c] = f2h_small_int((x * 7 + c * 3) % 17 - 8);
    uint16_t *dq, *dv, *dk, *dat;
    CHECK(hipMalloc((void**)&dq, zq.size() * 2) == 0 && hipMalloc((void**)&dv, vv.size() * 2) == 0 &&
          hipMalloc((void**)&dk, vv.size() * 2) == 0 && hipMalloc((void**)&dat, oo.size() * 2) == 0);
    hipMemcpy(dq, zq.data(), zq.size() * 2, 1); hipMemcpy(dv, vv.data(), vv.size() * 2, 1);
    hipMemcpy(dk, vv.data(), vv.size() * 2, 1);
    TensorView<f16> av(dat, TensorLayout::row_major({(size_t)M, (size_t)K}));
    TensorView<const f16> qv(dq, TensorLayout::row_major({(size_t)M, (size_t)K}));
    TensorView<const f16> kv(dk, TensorLayout::row_major({(size_t)NK, (size_t)K}));
    TensorView<const f16> vv_(dv, TensorLayout::row_major({(size_t)NK, (size_t)K}));
    tr.attention_f16(av, qv, kv, vv_, 0.125f, 1.0f, MatmulMask::None);
    CHECK(hipDeviceSynchronize() == 0);
    hipMemcpy(oo.data(), dat, oo.size() * 2, 2);
    int bad = 0;
    for (int c = 0; c < K; c++) {
      int sum = 0;
      for (int x = 0; x < NK; x++) sum += h2i(vv[(size_t)x * K + c]);
      for (int y = 0; y < M; y++) bad += h2d(oo[(size_t)y * K + c]) != (double)sum / NK;
    }
    CHECK(bad == 0);
    CHECK(throws([&] { tr.attention_f16(av, qv, kv.permute({1, 0}), vv_, 0.125f, 1.0f, MatmulMask::None); }));
  }
  {
    // GpuKernels with a workspace: a product with few tiles and a long K is split over K and
    // must give the bits of the unsplit call (inputs in {-1, 0, 1}: every sum is exact)
    const int M2 = 100, K2 = 1472, N2 = 1000;
    const int64_t need = adr_matmul_f16_workspace_bytes(1, M2, K2, N2, 1, N2, 0, 1, K2, 0, K2, 1, 0, 0, 0, 0);
    CHECK(need > 0);
    std::vector<uint16_t> a2((size_t)M2 * K2), w2((size_t)N2 * K2), o1((size_t)M2 * N2), o2((size_t)M2 * N2);
    for (auto& v : a2) v = f2h_small_int(rnd() % 2);
    for (auto& v : w2) v = f2h_small_int(rnd() % 2);
    uint16_t *da2, *dw2, *do1, *do2;
    void* ws;
    CHECK(hipMalloc((void**)&da2, a2.size() * 2) == 0 && hipMalloc((void**)&dw2, w2.size() * 2) == 0 &&
          hipMalloc((void**)&do1, o1.size() * 2) == 0 && hipMalloc((void**)&do2, o2.size() * 2) == 0 &&
          hipMalloc(&ws, (size_t)need) == 0);
    hipMemcpy(da2, a2.data(), a2.size() * 2, 1); hipMemcpy(dw2, w2.data(), w2.size() * 2, 1);
    GpuKernels with_ws(nullptr, ws, need);
    TensorView<f16> ov1(do1, TensorLayout::row_major({(size_t)M2, (size_t)N2}));
    TensorView<f16> ov2(do2, TensorLayout::row_major({(size_t)M2, (size_t)N2}));
    TensorView<const f16> lv2(da2, TensorLayout::row_major({(size_t)M2, (size_t)K2}));
    TensorView<const f16> wv2(dw2, TensorLayout::row_major({(size_t)N2, (size_t)K2}));
    gk.matmul_f16(ov1, lv2, wv2.permute({1, 0}), MatmulOptions::make());
    with_ws.matmul_f16(ov2, lv2, wv2.permute({1, 0}), MatmulOptions::make());
    CHECK(hipDeviceSynchronize() == 0);
    hipMemcpy(o1.data(), do1, o1.size() * 2, 2); hipMemcpy(o2.data(), do2, o2.size() * 2, 2);
    CHECK(o1 == o2);
    int ref = 0;
    for (int k = 0; k < K2; k++) ref += h2i(a2[(size_t)7 * K2 + k]) * h2i(w2[(size_t)9 * K2 + k]);
    CHECK(h2i(o2[(size_t)7 * N2 + 9]) == ref);
  }
  uint16_t bias = 0;
  CHECK(throws([&] { tr.matmul_f16(ov, lv, wv.permute({1, 0}), MatmulOptions::make().store(MatmulStore::GeluBias(&bias))); }));
}

// One line per tensor: name dtype rank shape.. stride.. begin end fnv1a64(bytes).  The Python
// test compares these with what torch's own loader returns for the same file.
static void dump_tensor(const std::string& name, const PickledModel& m, const PickledTensor& t) {
  static const char* names[] = {"i8", "i64", "f16", "f32", "f64"};
  uint64_t h = 1469598103934665603ull;
  for (size_t i = t.begin; i < t.end; i++) h = (h ^ m.mapping.data()[i]) * 1099511628211ull;
  printf("%s %s %zu", name.c_str(), names[(int)t.dtype], t.shape.size());
  for (size_t d : t.shape) printf(" %zu", d);
  for (size_t d : t.stride) printf(" %zu", d);
  printf(" %zu %zu %016llx\n", t.begin, t.end, (unsigned long long)h);
}

static int pickle_dump(int argc, char** argv) {
  try {
    if (!strcmp(argv[1], "pickle")) {
      auto m = PickledModel::load_file(argv[2], argc > 3 ? argv[3] : nullptr);
      for (auto& kv : m->tensors) dump_tensor(kv.first, *m, kv.second);
    } else {
      auto m = ShardedModel::load_huggingface(argv[2]);
      printf("shards %zu\n", m->shard_count());
      for (int i = 3; i < argc; i++) {
        auto f = m->find(argv[i]);
        dump_tensor(argv[i], *f.first, *f.second);
      }
    }
  } catch (const std::exception& e) {
    printf("ERROR %s\n", e.what());
    return 2;
  }
  return 0;
}

// Every weight of a LLaMA checkpoint through the model loaders (llama.rs:171-243), one line per
// address: name dtype rank shape.. stride.. bytes fnv1a64(bytes).
static void dump_loaded(const std::string& name, const LoadedTensor& t) {
  static const char* names[] = {"i8", "i64", "f16", "f32", "f64"};
  uint64_t h = 1469598103934665603ull;
  for (size_t i = 0; i < t.bytes; i++) h = (h ^ t.data[i]) * 1099511628211ull;
  printf("%s %s %zu", name.c_str(), names[(int)t.dtype], t.shape.size());
  for (size_t d : t.shape) printf(" %zu", d);
  for (size_t d : t.stride) printf(" %zu", d);
  printf(" %zu %016llx\n", t.bytes, (unsigned long long)h);
}

template <typename Names, typename Loader>
static void dump_llama(const Loader& loader, size_t layers) {
  auto one = [&](const LlamaModelAddress& a) { dump_loaded(Names::resolve(a), loader.load_tensor(a)); };
  one(LlamaModelAddress::token_embedding());
  for (size_t l = 0; l < layers; l++) {
    using B = LlamaTransformerBlockAddress;
    one(LlamaModelAddress::in_layer(l, B::attention_norm()));
    for (auto a : {LlamaAttentionAddress::Query, LlamaAttentionAddress::Key, LlamaAttentionAddress::Value,
                   LlamaAttentionAddress::Out})
      one(LlamaModelAddress::in_layer(l, B::of(a)));
    one(LlamaModelAddress::in_layer(l, B::mlp_norm()));
    for (auto a : {LlamaMLPAddress::Gate, LlamaMLPAddress::Expand, LlamaMLPAddress::Contract})
      one(LlamaModelAddress::in_layer(l, B::of(a)));
  }
  one(LlamaModelAddress::output_norm());
  one(LlamaModelAddress::token_projection());
}

// llama-meta <file> <layers> | llama-hf <dir> <layers> <dim> <n_heads>
static int llama_dump(int argc, char** argv) {
  try {
    const size_t layers = (size_t)atoll(argv[3]);
    if (!strcmp(argv[1], "llama-meta")) {
      auto m = PickledModel::load_file(argv[2]);
      dump_llama<MetaTensorNames>(MetaLlamaModelLoader(*m), layers);
    } else {
      if (argc < 6) throw std::runtime_error("usage: llama-hf dir layers dim n_heads");
      auto m = ShardedModel::load_huggingface(argv[2]);
      dump_llama<HuggingFaceTensorNames>(
          HuggingFaceLlamaModelLoader(*m, {(size_t)atoll(argv[4]), (size_t)atoll(argv[5])}), layers);
    }
  } catch (const std::exception& e) {
    printf("ERROR %s\n", e.what());
    return 2;
  }
  return 0;
}

// Checkpoint -> device -> u8: uploads one fp16 [N, K] tensor of the file, quantises it with
// adr_quantize_absmax_u8 and dequantises it again; prints the largest |x - dq(q(x))| / scale.
static int pickle_quantize(const char* path, const char* name, int block_size) {
  void* hip = dlopen("libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
  if (!hip) { printf("ERROR no hip runtime\n"); return 2; }
  auto hipMalloc = (int (*)(void**, size_t))dlsym(hip, "hipMalloc");
  auto hipMemcpy = (int (*)(void*, const void*, size_t, int))dlsym(hip, "hipMemcpy");
  auto hipDeviceSynchronize = (int (*)())dlsym(hip, "hipDeviceSynchronize");
  try {
    auto m = PickledModel::load_file(path);
    const PickledTensor& t = m->tensor(name);
    if (t.dtype != TensorDataType::F16 || t.shape.size() != 2 || t.stride[1] != 1 || t.stride[0] != t.shape[1])
      throw std::runtime_error("expected a contiguous fp16 matrix");
    const int rows = (int)t.shape[0], cols = (int)t.shape[1];
    const size_t n = (size_t)rows * cols;
    uint16_t *dx, *ds, *dy;
    uint8_t* dq;
    if (hipMalloc((void**)&dx, n * 2) || hipMalloc((void**)&dy, n * 2) || hipMalloc((void**)&dq, n) ||
        hipMalloc((void**)&ds, n / block_size * 2))
      throw std::runtime_error("hipMalloc failed");
    hipMemcpy(dx, m->bytes(t), n * 2, 1);  // the copy of load_tensor (pickle.rs:331-335)
    int rc = adr_quantize_absmax_u8(nullptr, dq, ds, dx, rows, cols, block_size);
    if (!rc) rc = adr_dequantize_absmax_u8(nullptr, dy, dq, ds, rows, cols, block_size);
    if (rc || hipDeviceSynchronize()) throw std::runtime_error("launch failed");
    std::vector<uint16_t> y(n), sc(n / block_size);
    hipMemcpy(y.data(), dy, n * 2, 2);
    hipMemcpy(sc.data(), ds, sc.size() * 2, 2);
    const uint16_t* x = (const uint16_t*)m->bytes(t);
    double worst = 0;
    for (size_t i = 0; i < n; i++) {
      const double s = h2d(sc[i / block_size]);
      if (s > 0) worst = std::max(worst, std::fabs(h2d(x[i]) - h2d(y[i])) / s);
    }
    printf("rows %d cols %d worst_error_in_scales %.4f\n", rows, cols, worst);
  } catch (const std::exception& e) {
    printf("ERROR %s\n", e.what());
    return 2;
  }
  return 0;
}

int main(int argc, char** argv) {
  if (argc > 2 && (!strcmp(argv[1], "pickle") || !strcmp(argv[1], "sharded"))) return pickle_dump(argc, argv);
  if (argc > 3 && (!strcmp(argv[1], "llama-meta") || !strcmp(argv[1], "llama-hf"))) return llama_dump(argc, argv);
  if (argc > 4 && !strcmp(argv[1], "quantize")) return pickle_quantize(argv[2], argv[3], atoi(argv[4]));
  if (argc > 1 && !strcmp(argv[1], "gpu")) gpu_test(); else cpu_tests();
  printf(failures ? "FAILED (%d)\n" : "OK\n", failures);
  return failures != 0;
}
