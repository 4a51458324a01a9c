// Test driver of the C++ layer shims: builds the layers by weight name through the test harness that stands in for
// KsanaLLM's layer factory, runs Forward on the device and writes the result for the Python parity tests.
//
//   layer_driver w4a16 <dir> <f16|bf16> <m> <k> <n> <g> <gptq|awq> <gptq|awq|rowmajor> <none|awq|uint8|additive>
//       reads <dir>/qweight.bin, qzeros.bin (unless none), scales.bin, act.bin; writes <dir>/out.bin
//   layer_driver fp8 <dir> <f16|bf16|f32> <m> <k> <n> <wscales: 1|n> <static: 0|1>
//   layer_driver fp8load <dir> <f16|bf16> <m> <k> <nq> <nkv> <per_channel: 0|1>
//     q/k/v weights [k, n*] T from wq_src.bin / wk_src.bin / wv_src.bin: converted per tensor, fused, scales merged
//       reads <dir>/wq.bin, wscale.bin, act.bin, iscale.bin (static); writes <dir>/out.bin
//   layer_driver errors
//       exercises the error conventions; prints one line per check
// Prints "OK <m> <n> <dtype>" or "THROW <message>".
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "ksq.h"
#include "layer_harness.h"

using namespace ksana_llm;

static std::vector<char> ReadFile(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) throw std::runtime_error("cannot open " + path);
  return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static Tensor Upload(const std::vector<char>& bytes, DataType dtype, const std::vector<size_t>& shape) {
  Tensor t;
  CreateTensor(t, shape, dtype, 0, MEMORY_DEVICE);
  if (t.GetTotalBytes() != bytes.size())
    throw std::runtime_error("size mismatch: file has " + std::to_string(bytes.size()) + " bytes, tensor " +
                             std::to_string(t.GetTotalBytes()));
  if (hipMemcpy(t.GetPtr<void>(), bytes.data(), bytes.size(), hipMemcpyHostToDevice) != hipSuccess)
    throw std::runtime_error("hipMemcpy H2D failed");
  return t;
}

static void Download(const Tensor& t, const std::string& path) {
  std::vector<char> host(t.GetTotalBytes());
  if (hipDeviceSynchronize() != hipSuccess) throw std::runtime_error("device error after Forward");
  if (hipMemcpy(host.data(), t.GetPtr<void>(), host.size(), hipMemcpyDeviceToHost) != hipSuccess)
    throw std::runtime_error("hipMemcpy D2H failed");
  std::ofstream f(path, std::ios::binary);
  f.write(host.data(), host.size());
}

struct OneWeight : public BaseWeight {
  Tensor t;
  Tensor GetModelWeights(const std::string&) override { return t; }
};

template <typename T>
static int RunW4(int argc, char** argv) {
  const std::string dir = argv[2];
  const size_t m = atol(argv[4]), k = atol(argv[5]), n = atol(argv[6]), g = atol(argv[7]);
  const std::string method = argv[8], layout = argv[9], zeros = argv[10];
  // none | desc | silu | bias | parts:n0:n1:.. | adopt (no load-time repack: the loader's own tensors reach Forward)
  const std::string extra = argc > 11 ? argv[11] : "none";
  const DataType dt = TypeTraits<T>::kDataType;
  auto context = std::make_shared<Context>(1);

  Tensor scales = Upload(ReadFile(dir + "/scales.bin"), dt, {k / g, n});
  Tensor qweight, qzeros, weight, weight_sz;
  GroupWeightLayout lay;
  if (layout == "gptq") {
    lay = GROUP_WEIGHT_GPTQ_INT32;
    qweight = Upload(ReadFile(dir + "/qweight.bin"), TYPE_INT32, {k / 8, n});
  } else if (layout == "awq") {
    lay = GROUP_WEIGHT_AWQ_INT32;
    qweight = Upload(ReadFile(dir + "/qweight.bin"), TYPE_INT32, {k, n / 8});
  } else {
    lay = layout == "cutlass80" ? GROUP_WEIGHT_CUTLASS_SM80 : layout == "cutlass90" ? GROUP_WEIGHT_CUTLASS_SM90
                                                                                  : GROUP_WEIGHT_ROWMAJOR_INT4;
    qweight = Upload(ReadFile(dir + "/qweight.bin"), TYPE_INT8, {k, n / 2});
  }
  const Tensor* zp = nullptr;
  bool additive = false;
  if (zeros == "awq") {
    qzeros = Upload(ReadFile(dir + "/qzeros.bin"), TYPE_INT32, {k / g, n / 8});
    zp = &qzeros;
  } else if (zeros == "uint8") {
    qzeros = Upload(ReadFile(dir + "/qzeros.bin"), TYPE_UINT8, {k / g, n});
    zp = &qzeros;
  } else if (zeros == "additive") {
    qzeros = Upload(ReadFile(dir + "/qzeros.bin"), dt, {k / g, n});
    zp = &qzeros;
    additive = true;
  }
  Tensor perm;
  if (extra == "desc") {
    // what a loader does with a desc_act checkpoint: sort g_idx on the host, keep the permutation on the device
    std::vector<char> raw = ReadFile(dir + "/g_idx.bin");
    std::vector<int32_t> g_idx(raw.size() / 4), order;
    memcpy(g_idx.data(), raw.data(), raw.size());
    SortGptqGIdx(g_idx, g, order);
    std::vector<char> bytes(order.size() * 4);
    memcpy(bytes.data(), order.data(), bytes.size());
    perm = Upload(bytes, TYPE_INT32, {k});
  }
  std::vector<Tensor> part_tensors;  // qweight, qzeros, scales of every part (kept alive until the repack ran)
  if (extra.rfind("parts:", 0) == 0) {
    // "parts:n0:n1:..": the AWQ checkpoint comes as separate tensors qweight_i.bin / qzeros_i.bin / scales_i.bin that
    // share K (q_proj, k_proj, v_proj); they are repacked side by side into one fused weight
    std::vector<size_t> widths;
    for (size_t pos = 6; pos < extra.size();) {
      const size_t end = extra.find(':', pos);
      widths.push_back(std::stoul(extra.substr(pos, end - pos)));
      pos = end == std::string::npos ? extra.size() : end + 1;
    }
    part_tensors.reserve(3 * widths.size());
    std::vector<GroupWeightPart> parts;
    for (size_t i = 0; i < widths.size(); ++i) {
      const std::string tag = "_" + std::to_string(i) + ".bin";
      part_tensors.push_back(Upload(ReadFile(dir + "/qweight" + tag), TYPE_INT32, {k, widths[i] / 8}));
      part_tensors.push_back(Upload(ReadFile(dir + "/qzeros" + tag), TYPE_INT32, {k / g, widths[i] / 8}));
      part_tensors.push_back(Upload(ReadFile(dir + "/scales" + tag), dt, {k / g, widths[i]}));
      const size_t base = part_tensors.size() - 3;
      parts.push_back({&part_tensors[base], &part_tensors[base + 1], &part_tensors[base + 2], widths[i]});
    }
    RepackFusedGroupQuantWeight(GROUP_WEIGHT_AWQ_INT32, parts, false, k, g, weight, weight_sz, 0,
                                context->GetComputeStreams()[0]);
  } else if (extra == "adopt") {
    // what KsanaLLM's own loader hands the layer: "*.weight" as its back end preprocessed it, with `.scales` and the
    // additive `.zeros` bound (KS/models/quant/quant_weight.cpp:632-636); the layer converts it at its first Forward
    weight = qweight;
    weight.dtype = TYPE_I4_GROUP;
    weight.scales = &scales;
    weight.zeros = const_cast<Tensor*>(zp);
  } else {
    RepackGroupQuantWeight(lay, qweight, zp, additive, scales, k, n, g, weight, weight_sz, 0,
                           context->GetComputeStreams()[0], extra == "desc" ? &perm : nullptr, extra == "silu");
  }

  ModelConfig cfg;
  cfg.is_quant = true;
  cfg.quant_config.method = method == "awq" ? QUANT_AWQ : QUANT_GPTQ;
  cfg.quant_config.group_size = g;
  cfg.quant_config.desc_act = extra == "desc";
  cfg.hidden_units = k;
  cfg.size_per_head = n;  // query_key_value: k = hidden_units, n = size_per_head * (head_num + 2 * kv heads)
  cfg.head_num = 1;
  cfg.num_key_value_heads = 0;
  cfg.max_scheduler_token_num = m;
  LayerHarness<T> factory(cfg, context);
  auto holder = std::make_shared<OneWeight>();
  holder->t = weight;
  auto layer = factory.ForWeight(*holder, "model.layers.0.self_attn.query_key_value.weight", dt);

  if (extra == "adopt") {
    auto group = std::dynamic_pointer_cast<GroupMatMulLayer<T, TYPE_I4_GROUP>>(layer);
    if (!group) throw std::runtime_error("harness did not build a GroupMatMulLayer");
    group->SetLoaderLayout(lay);
  }
  Tensor bias;
  if (extra == "silu" || extra == "bias") {
    auto group = std::dynamic_pointer_cast<GroupMatMulLayer<T, TYPE_I4_GROUP>>(layer);
    if (!group) throw std::runtime_error("harness did not build a GroupMatMulLayer");
    if (extra == "bias") {
      bias = Upload(ReadFile(dir + "/bias.bin"), dt, {n});
      group->SetEpilogue(KSQ_EPILOGUE_BIAS, &bias);
    } else {
      group->SetEpilogue(KSQ_EPILOGUE_SILU_MUL);
    }
  }

  Tensor act = Upload(ReadFile(dir + "/act.bin"), dt, {m, k});
  Tensor out;
  CreateTensor(out, {m, n}, dt, 0, MEMORY_DEVICE);
  out.shape = {0};
  std::vector<Tensor> outputs = {out};
  Status st = layer->Forward({act, weight}, outputs);
  if (!st.OK()) throw std::runtime_error("Forward returned " + st.GetMessage());
  if (extra == "adopt") {  // the second call finds the converted weight: same tensor, nothing to do
    st = layer->Forward({act, weight}, outputs);
    if (!st.OK()) throw std::runtime_error("second Forward returned " + st.GetMessage());
    ForgetAdoptedGroupQuantWeights(0);
  }
  Download(outputs[0], dir + "/out.bin");
  std::cout << "OK " << outputs[0].shape[0] << " " << outputs[0].shape[1] << " " << outputs[0].dtype << std::endl;
  return 0;
}

template <typename T>
static int RunFp8(int argc, char** argv) {
  const std::string dir = argv[2];
  const size_t m = atol(argv[4]), k = atol(argv[5]), n = atol(argv[6]);
  const size_t nws = std::string(argv[7]) == "n" ? n : 1;
  const bool is_static = atoi(argv[8]) != 0;
  const DataType dt = TypeTraits<T>::kDataType;
  auto context = std::make_shared<Context>(1);
  Tensor wq = Upload(ReadFile(dir + "/wq.bin"), TYPE_FP8_E4M3, {n, k});
  Tensor wscale = Upload(ReadFile(dir + "/wscale.bin"), TYPE_FP32, {nws});
  Tensor iscale;
  wq.weight_scales = &wscale;
  if (is_static) {
    iscale = Upload(ReadFile(dir + "/iscale.bin"), TYPE_FP32, {1});
    wq.input_scales = &iscale;
  }
  ModelConfig cfg;
  cfg.max_scheduler_token_num = m;
  LayerHarness<T> factory(cfg, context);
  auto holder = std::make_shared<OneWeight>();
  holder->t = wq;
  auto layer = factory.ForWeight(*holder, "model.layers.0.mlp.down_proj.weight", dt);
  Tensor act = Upload(ReadFile(dir + "/act.bin"), dt, {m, k});
  Tensor out;
  CreateTensor(out, {m, n}, dt, 0, MEMORY_DEVICE);
  std::vector<Tensor> outputs = {out};
  Status st = layer->Forward({act, wq}, outputs);
  if (!st.OK()) throw std::runtime_error("Forward returned " + st.GetMessage());
  Download(outputs[0], dir + "/out.bin");
  std::cout << "OK " << outputs[0].shape[0] << " " << outputs[0].shape[1] << " " << outputs[0].dtype << std::endl;
  return 0;
}

// The load-time path of an FP8 checkpoint that stores q, k and v separately: convert each [k, n] weight on the fly
// (one scale per tensor), put the three [n, k] results one after another, merge the scales, run the layer.
template <typename T>
static int RunFp8Load(int argc, char** argv) {
  const std::string dir = argv[2];
  const size_t m = atol(argv[4]), k = atol(argv[5]), nq = atol(argv[6]), nkv = atol(argv[7]);
  const bool per_channel = atoi(argv[8]) != 0;
  const DataType dt = TypeTraits<T>::kDataType;
  auto context = std::make_shared<Context>(1);
  Stream& stream = context->GetComputeStreams()[0];
  const size_t n = nq + 2 * nkv;
  Tensor fused;
  CreateTensor(fused, {n, k}, TYPE_FP8_E4M3, 0, MEMORY_DEVICE);
  const char* names[3] = {"/wq_src.bin", "/wk_src.bin", "/wv_src.bin"};
  const size_t rows[3] = {nq, nkv, nkv};
  Tensor part_fp8[3], part_scale[3];
  size_t row0 = 0;
  for (int i = 0; i < 3; ++i) {
    Tensor src = Upload(ReadFile(dir + names[i]), dt, {k, rows[i]});
    ConvertFp8Weight(src, false, part_fp8[i], part_scale[i], 0, stream);
    if (hipMemcpyAsync(fused.GetPtr<char>() + row0 * k, part_fp8[i].GetPtr<void>(), rows[i] * k, hipMemcpyDeviceToDevice,
                       static_cast<hipStream_t>(stream.Get())) != hipSuccess)
      throw std::runtime_error("hipMemcpyAsync failed");
    row0 += rows[i];
  }
  Tensor merged;
  MergeFp8QkvScales(fused, part_scale[0], part_scale[1], part_scale[2], nq, nkv, nkv, per_channel, merged, 0, stream);
  if (hipStreamSynchronize(static_cast<hipStream_t>(stream.Get())) != hipSuccess) throw std::runtime_error("sync failed");
  Download(fused, dir + "/fused.bin");
  Download(merged, dir + "/merged_scale.bin");

  ModelConfig cfg;
  cfg.max_scheduler_token_num = m;
  LayerHarness<T> factory(cfg, context);
  auto holder = std::make_shared<OneWeight>();
  holder->t = fused;
  auto layer = factory.ForWeight(*holder, "model.layers.0.self_attn.query_key_value.weight", dt);
  Tensor act = Upload(ReadFile(dir + "/act.bin"), dt, {m, k});
  Tensor out;
  CreateTensor(out, {m, n}, dt, 0, MEMORY_DEVICE);
  std::vector<Tensor> outputs = {out};
  Status st = layer->Forward({act, fused}, outputs);
  if (!st.OK()) throw std::runtime_error("Forward returned " + st.GetMessage());
  Download(outputs[0], dir + "/out.bin");
  std::cout << "OK " << outputs[0].shape[0] << " " << outputs[0].shape[1] << " " << outputs[0].dtype << std::endl;
  return 0;
}

template <typename F>
static void Expect(const char* name, bool want_throw, F f) {
  bool threw = false;
  std::string msg;
  try {
    f();
  } catch (const std::runtime_error& e) {
    threw = true;
    msg = e.what();
  } catch (const std::bad_any_cast& e) {
    threw = true;
    msg = std::string("bad_any_cast: ") + e.what();
  }
  std::cout << (threw == want_throw ? "PASS " : "FAIL ") << name << (threw ? " :: " + msg : "") << std::endl;
}

static int RunErrors() {
  auto context = std::make_shared<Context>(1);
  ModelConfig cfg;
  cfg.is_quant = true;
  cfg.quant_config.method = QUANT_GPTQ;
  LayerHarness<float16> factory(cfg, context);
  std::vector<std::any> good = {false, false, true, CUTLASS_BACKEND, size_t(16), size_t(256), size_t(256), size_t(128), true};

  Expect("activation type without a layer class throws", true,
         [&] { factory.Make(TYPE_I4_GROUP, TYPE_FP32, good); });
  Expect("parameter pack in the wrong order throws", true, [&] {
    std::vector<std::any> bad = {size_t(16), false, true};
    factory.Make(TYPE_I4_GROUP, TYPE_FP16, bad);
  });
  Expect("group size 32 is refused when the workspace is sized", true, [&] {
    std::vector<std::any> p = good;
    p[7] = size_t(32);
    auto l = factory.Make(TYPE_I4_GROUP, TYPE_FP16, p);
    Tensor a, w, s, o;
    CreateTensor(a, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    CreateTensor(w, {256, 128}, TYPE_UINT8, 0, MEMORY_DEVICE);
    CreateTensor(s, {8, 256}, TYPE_UINT32, 0, MEMORY_DEVICE);
    CreateTensor(o, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    w.scales = &s;
    std::vector<Tensor> outs = {o};
    l->Forward({a, w}, outs);
  });
  Expect("k not a whole number of groups is refused", true, [&] {
    std::vector<std::any> p = good;
    p[6] = size_t(192);
    factory.Make(TYPE_I4_GROUP, TYPE_FP16, p);
  });
  Expect("desc_act weight without a bound perm throws at Forward", true, [&] {
    std::vector<std::any> p = good;
    p[1] = true;
    auto l = factory.Make(TYPE_I4_GROUP, TYPE_FP16, p);
    Tensor a, w, s, o;
    CreateTensor(a, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    CreateTensor(w, {256, 128}, TYPE_UINT8, 0, MEMORY_DEVICE);
    CreateTensor(s, {2, 256}, TYPE_UINT32, 0, MEMORY_DEVICE);
    CreateTensor(o, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    w.scales = &s;
    std::vector<Tensor> outs = {o};
    l->Forward({a, w}, outs);
  });
  Expect("weight without bound scales throws", true, [&] {
    auto l = factory.Make(TYPE_I4_GROUP, TYPE_FP16, good);
    Tensor a, w, o;
    CreateTensor(a, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    CreateTensor(w, {256, 128}, TYPE_UINT8, 0, MEMORY_DEVICE);
    CreateTensor(o, {1, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    std::vector<Tensor> outs = {o};
    l->Forward({a, w}, outs);
  });
  Expect("fp8: null weight scale throws", true, [&] {
    std::vector<std::any> p = {size_t(4), size_t(256)};
    auto l = factory.Make(TYPE_FP8_E4M3, TYPE_FP16, p);
    Tensor a, w, o;
    CreateTensor(a, {4, 256}, TYPE_FP16, 0, MEMORY_DEVICE);
    CreateTensor(w, {64, 256}, TYPE_FP8_E4M3, 0, MEMORY_DEVICE);
    CreateTensor(o, {4, 64}, TYPE_FP16, 0, MEMORY_DEVICE);
    std::vector<Tensor> outs = {o};
    l->Forward({a, w}, outs);
  });
  Expect("fp8: workspace smaller than the request throws", true, [&] {
    std::vector<std::any> p = {size_t(4), size_t(256)};
    auto l = factory.Make(TYPE_FP8_E4M3, TYPE_FP16, p);
    Tensor a, w, o, sc;
    CreateTensor(a, {64, 256}, TYPE_FP16, 0, MEMORY_DEVICE);  // m = 64 > max_m = 4
    CreateTensor(w, {64, 256}, TYPE_FP8_E4M3, 0, MEMORY_DEVICE);
    CreateTensor(sc, {1}, TYPE_FP32, 0, MEMORY_DEVICE);
    CreateTensor(o, {64, 64}, TYPE_FP16, 0, MEMORY_DEVICE);
    w.weight_scales = &sc;
    std::vector<Tensor> outs = {o};
    l->Forward({a, w}, outs);
  });
  Expect("well-formed group layer builds and shares one workspace", false, [&] {
    auto l1 = factory.Make(TYPE_I4_GROUP, TYPE_FP16, good);
    std::vector<std::any> big = good;
    big[5] = size_t(4096);
    big[6] = size_t(4096);
    auto l2 = factory.Make(TYPE_I4_GROUP, TYPE_FP16, big);
    if (!factory.Workspace() || factory.Workspace()->GetTotalBytes() < l2->GetWorkSpaceSize())
      throw std::runtime_error("shared workspace was not grown to the largest request");
  });
  return 0;
}

int main(int argc, char** argv) {
  try {
    if (argc >= 2 && std::string(argv[1]) == "errors") return RunErrors();
    if ((argc == 11 || argc == 12) && std::string(argv[1]) == "w4a16")
      return std::string(argv[3]) == "f16" ? RunW4<float16>(argc, argv) : RunW4<bfloat16>(argc, argv);
    if (argc == 9 && std::string(argv[1]) == "fp8")
      return std::string(argv[3]) == "f16"   ? RunFp8<float16>(argc, argv)
             : std::string(argv[3]) == "f32" ? RunFp8<float>(argc, argv)
                                             : RunFp8<bfloat16>(argc, argv);
    if (argc == 9 && std::string(argv[1]) == "fp8load")
      return std::string(argv[3]) == "f16" ? RunFp8Load<float16>(argc, argv) : RunFp8Load<bfloat16>(argc, argv);
    std::cerr << "usage: see the header of layer_driver.cpp" << std::endl;
    return 2;
  } catch (const std::exception& e) {
    std::cout << "THROW " << e.what() << std::endl;
    return 1;
  }
}
