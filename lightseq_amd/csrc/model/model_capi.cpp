// extern "C" wrapper of the LSModel interface: exceptions -> status codes.
#include <string.h>

#include <memory>

#include "../../../include/lightseq_model.h"
#include "../ls_launch.h"
#include "ls_model.h"
#include "quant_bert.h"
#include "quant_gpt.h"
#include "quant_transformer.h"

using lightseq::hip::LSModel;
using lightseq::hip::LSModelFactory;
using lightseq::hip::QuantBert;
using lightseq::hip::QuantBertEncoder;
using lightseq::hip::QuantGpt;
using lightseq::hip::QuantTransformer;

struct ls_model {
  std::unique_ptr<LSModel> impl;
  std::string name_buf;
};

namespace {

template <typename F>
int guarded(F&& f) {
  try {
    f();
    return LSH_OK;
  } catch (const std::exception& e) {
    return lsh::lsh_fail(LSH_ERR_INVALID, e.what());
  } catch (...) {
    return lsh::lsh_fail(LSH_ERR_INVALID, "unknown C++ exception");
  }
}

int copy_shape(const std::vector<int>& v, int* shape, int* ndim) {
  if (!shape || !ndim) return lsh::lsh_fail(LSH_ERR_INVALID, "null shape pointer");
  if (v.size() > LS_MAX_DIMS) return lsh::lsh_fail(LSH_ERR_INVALID, "too many dimensions");
  *ndim = (int)v.size();
  for (size_t i = 0; i < v.size(); ++i) shape[i] = v[i];
  return LSH_OK;
}

#define NEED_MODEL(m) \
  if (!(m) || !(m)->impl) return lsh::lsh_fail(LSH_ERR_INVALID, "null model handle")

}  // namespace

extern "C" {

int ls_model_create(const char* class_name, const char* weight_path, int max_batch_size,
                    ls_model** model) {
  if (!class_name || !weight_path || !model)
    return lsh::lsh_fail(LSH_ERR_INVALID, "ls_model_create: null argument");
  *model = nullptr;
  return guarded([&] {
    LSModel* p = LSModelFactory::GetInstance().CreateModel(class_name, weight_path, max_batch_size);
    *model = new ls_model{std::unique_ptr<LSModel>(p), {}};
  });
}

int ls_model_destroy(ls_model* model) {
  if (!model) return LSH_OK;
  return guarded([&] { delete model; });
}

int ls_model_infer(ls_model* model) {
  NEED_MODEL(model);
  return guarded([&] { model->impl->Infer(); });
}

int ls_model_set_input_ptr(ls_model* model, int index, void* input_ptr) {
  NEED_MODEL(model);
  return guarded([&] { model->impl->set_input_ptr(index, input_ptr); });
}

int ls_model_set_input_shape(ls_model* model, int index, const int* shape, int ndim) {
  NEED_MODEL(model);
  if (!shape || ndim < 0 || ndim > LS_MAX_DIMS)
    return lsh::lsh_fail(LSH_ERR_INVALID, "ls_model_set_input_shape: bad shape");
  return guarded([&] { model->impl->set_input_shape(index, std::vector<int>(shape, shape + ndim)); });
}

int ls_model_get_input_max_shape(ls_model* model, int index, int* shape, int* ndim) {
  NEED_MODEL(model);
  int rc = LSH_OK;
  int g = guarded([&] { rc = copy_shape(model->impl->get_input_max_shape(index), shape, ndim); });
  return g ? g : rc;
}

int ls_model_get_input_size(ls_model* model, int* count) {
  NEED_MODEL(model);
  if (!count) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  *count = model->impl->get_input_size();
  return LSH_OK;
}

int ls_model_get_input_name(ls_model* model, int index, const char** name) {
  NEED_MODEL(model);
  if (!name) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  return guarded([&] {
    model->name_buf = model->impl->get_input_name(index);
    *name = model->name_buf.c_str();
  });
}

int ls_model_get_input_dtype(ls_model* model, int index, int* dtype) {
  NEED_MODEL(model);
  if (!dtype) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  return guarded([&] { *dtype = (int)model->impl->get_input_dtype(index); });
}

int ls_model_set_output_ptr(ls_model* model, int index, void* output_ptr) {
  NEED_MODEL(model);
  return guarded([&] { model->impl->set_output_ptr(index, output_ptr); });
}

int ls_model_get_output_ptr(ls_model* model, int index, const void** output_ptr) {
  NEED_MODEL(model);
  if (!output_ptr) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  return guarded([&] { *output_ptr = model->impl->get_output_ptr(index); });
}

int ls_model_get_output_size(ls_model* model, int* count) {
  NEED_MODEL(model);
  if (!count) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  *count = model->impl->get_output_size();
  return LSH_OK;
}

int ls_model_get_output_name(ls_model* model, int index, const char** name) {
  NEED_MODEL(model);
  if (!name) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  return guarded([&] {
    model->name_buf = model->impl->get_output_name(index);
    *name = model->name_buf.c_str();
  });
}

int ls_model_get_output_shape(ls_model* model, int index, int* shape, int* ndim) {
  NEED_MODEL(model);
  int rc = LSH_OK;
  int g = guarded([&] { rc = copy_shape(model->impl->get_output_shape(index), shape, ndim); });
  return g ? g : rc;
}

int ls_model_get_output_max_shape(ls_model* model, int index, int* shape, int* ndim) {
  NEED_MODEL(model);
  int rc = LSH_OK;
  int g = guarded([&] { rc = copy_shape(model->impl->get_output_max_shape(index), shape, ndim); });
  return g ? g : rc;
}

int ls_model_get_output_dtype(ls_model* model, int index, int* dtype) {
  NEED_MODEL(model);
  if (!dtype) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  return guarded([&] { *dtype = (int)model->impl->get_output_dtype(index); });
}

int ls_model_benchmark_mode(ls_model* model, int is_benchmark) {
  NEED_MODEL(model);
  return guarded([&] { model->impl->benchmark_mode(is_benchmark != 0); });
}

int ls_model_get_stream(ls_model* model, lsh_stream_t* stream) {
  NEED_MODEL(model);
  if (!stream) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  *stream = reinterpret_cast<lsh_stream_t>(model->impl->get_stream());
  return LSH_OK;
}

// the encoder stack of either model class, or nullptr
static QuantBertEncoder* encoder_of(ls_model* model) {
  if (QuantBert* qb = dynamic_cast<QuantBert*>(model->impl.get())) return qb->encoder();
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get()))
    return qt->encoder();
  return nullptr;
}

int ls_model_set_profiling(ls_model* model, int on) {
  NEED_MODEL(model);
  QuantBertEncoder* enc = encoder_of(model);
  if (!enc) return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "this model has no profiled encoder stack");
  return guarded([&] {
    enc->set_profiling(on != 0);
    enc->reset_profile();
  });
}

int ls_model_get_profile(ls_model* model, char* buf, int capacity) {
  NEED_MODEL(model);
  QuantBertEncoder* enc = encoder_of(model);
  if (!enc) return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "this model has no profiled encoder stack");
  if (!buf || capacity <= 0) return lsh::lsh_fail(LSH_ERR_INVALID, "null buffer");
  std::string out = "[";
  bool first = true;
  for (const auto& p : enc->profile()) {
    if (!first) out += ",";
    first = false;
    out += "{\"site\":\"" + p.site + "\",\"kernel\":\"" + p.kernel + "\",\"m\":" +
           std::to_string(p.m) + ",\"n\":" + std::to_string(p.n) + ",\"k\":" +
           std::to_string(p.k) + ",\"launches\":" + std::to_string(p.launches) +
           ",\"total_ms\":" + std::to_string(p.total_ms) + "}";
  }
  out += "]";
  if ((int)out.size() + 1 > capacity) return lsh::lsh_fail(LSH_ERR_INVALID, "buffer too small");
  memcpy(buf, out.c_str(), out.size() + 1);
  return LSH_OK;
}

int ls_model_set_tap(ls_model* model, int layer, const char* name, void* dst) {
  NEED_MODEL(model);
  if (!name) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  if (!strcmp(name, "enc_out")) {
    QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get());
    if (!qt) return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "enc_out is a QuantTransformer tap");
    qt->set_encoder_output_tap(static_cast<__half*>(dst));
    return LSH_OK;
  }
  // "dec.<name>": an intermediate of a generation step of QuantTransformer's decoder or of
  // QuantGpt (layer `layer`, at the step given to ls_model_set_tap_step)
  if (!strncmp(name, "dec.", 4)) {
    if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
      qg->encoder()->step_taps.set(layer, name + 4, dst);
      return LSH_OK;
    }
    if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get())) {
      qt->decoder()->step_taps.set(layer, name + 4, dst);
      return LSH_OK;
    }
    return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "step taps belong to QuantTransformer and QuantGpt");
  }
  QuantBertEncoder* enc = encoder_of(model);
  if (!enc) return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "this model has no tapped encoder stack");
  auto& t = enc->taps;
  t.tap_layer = layer;
  int8_t* p = static_cast<int8_t*>(dst);
  if (!strcmp(name, "ln1_q")) t.ln1_q = p;
  else if (!strcmp(name, "qkv_q")) t.qkv_q = p;
  else if (!strcmp(name, "ctx_q")) t.ctx_q = p;
  else if (!strcmp(name, "out_q")) t.out_q = p;
  else if (!strcmp(name, "ln2_q")) t.ln2_q = p;
  else if (!strcmp(name, "ffn1_q")) t.ffn1_q = p;
  else if (!strcmp(name, "act_q")) t.act_q = p;
  else if (!strcmp(name, "ffn2_acc")) t.ffn2_acc = static_cast<int32_t*>(dst);
  else if (!strcmp(name, "res_attn")) t.res_attn = static_cast<__half*>(dst);
  else if (!strcmp(name, "res_ffn")) t.res_ffn = static_cast<__half*>(dst);
  else return lsh::lsh_fail(LSH_ERR_INVALID, "unknown tap name");
  return LSH_OK;
}

int ls_model_set_tap_step(ls_model* model, int step) {
  NEED_MODEL(model);
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    qg->encoder()->step_taps.set_step(step);
    return LSH_OK;
  }
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get())) {
    qt->decoder()->step_taps.set_step(step);
    return LSH_OK;
  }
  return lsh::lsh_fail(LSH_ERR_UNSUPPORTED, "step taps belong to QuantTransformer and QuantGpt");
}

int ls_model_set_step_record(ls_model* model, int8_t* logits, int* alive_seq, int max_steps) {
  NEED_MODEL(model);
  if (max_steps < 0) return lsh::lsh_fail(LSH_ERR_INVALID, "negative max_steps");
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    qg->encoder()->set_step_record(logits, max_steps);
    return LSH_OK;
  }
  QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get());
  if (!qt)
    return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                         "step records are a debug aid of QuantTransformer and QuantGpt");
  qt->decoder()->set_step_record(logits, alive_seq, max_steps);
  return LSH_OK;
}

int ls_model_set_graph_mode(ls_model* model, int on) {
  NEED_MODEL(model);
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    qg->encoder()->graph_mode(on != 0);
    return LSH_OK;
  }
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get())) {
    qt->decoder()->graph_mode(on != 0);
    return LSH_OK;
  }
  return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                       "graph mode applies to the generation steps of QuantTransformer and QuantGpt");
}

int ls_model_set_seed(ls_model* model, unsigned long long seed) {
  NEED_MODEL(model);
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get()))
    return guarded([&] { qg->encoder()->set_seed(seed); });
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get()))
    return guarded([&] { qt->decoder()->set_seed(seed); });
  return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                       "a seed applies to the random sampling of QuantGpt and QuantTransformer");
}

int ls_model_get_graph_stats(ls_model* model, int* captured, long long* replayed) {
  NEED_MODEL(model);
  if (!captured || !replayed) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    *captured = qg->encoder()->graphs_captured();
    *replayed = qg->encoder()->graphs_replayed();
    return LSH_OK;
  }
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get())) {
    *captured = qt->decoder()->graphs_captured();
    *replayed = qt->decoder()->graphs_replayed();
    return LSH_OK;
  }
  return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                       "graph mode applies to the generation steps of QuantTransformer and QuantGpt");
}

int ls_model_get_graph_nodes(ls_model* model, int* nodes) {
  NEED_MODEL(model);
  if (!nodes) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    *nodes = qg->encoder()->graph_nodes();
    return LSH_OK;
  }
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get())) {
    *nodes = qt->decoder()->graph_nodes();
    return LSH_OK;
  }
  return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                       "graph mode applies to the generation steps of QuantTransformer and QuantGpt");
}

int ls_model_get_phase_times(ls_model* model, float* prepare_ms, float* steps_ms, int* steps) {
  NEED_MODEL(model);
  if (!prepare_ms || !steps_ms || !steps) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  const lightseq::hip::PhaseEvents* ph = nullptr;
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) ph = &qg->encoder()->phases();
  if (QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get()))
    ph = &qt->decoder()->phases();
  if (!ph)
    return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                         "phase times exist for the generation models QuantTransformer and QuantGpt");
  bool have = false;
  const int rc = guarded([&] { have = ph->times(prepare_ms, steps_ms, steps); });
  if (rc != LSH_OK) return rc;
  if (!have) return lsh::lsh_fail(LSH_ERR_INVALID, "no generation run has completed yet");
  return LSH_OK;
}

int ls_model_get_steps_run(ls_model* model, int* steps) {
  NEED_MODEL(model);
  if (!steps) return lsh::lsh_fail(LSH_ERR_INVALID, "null pointer");
  if (QuantGpt* qg = dynamic_cast<QuantGpt*>(model->impl.get())) {
    *steps = qg->encoder()->steps_run();
    return LSH_OK;
  }
  QuantTransformer* qt = dynamic_cast<QuantTransformer*>(model->impl.get());
  if (!qt)
    return lsh::lsh_fail(LSH_ERR_UNSUPPORTED,
                         "step records are a debug aid of QuantTransformer and QuantGpt");
  *steps = qt->decoder()->steps_run();
  return LSH_OK;
}

}  // extern "C"
