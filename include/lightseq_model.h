/*
 * lightseq_model.h -- C ABI of the model entry points (one MI355X, one stream).
 *
 * Replaces the C++ interface lightseq::cuda::LSModel / LSModelFactory of the
 * reference (lightseq/inference/pywrapper/model_base.h:59-148), which is what its
 * pybind module (pywrapper/wrapper.cc), C++ examples and Triton backend bind.
 * Every LSModel method has one function here with the same meaning; C++ exceptions
 * become a non-zero status and the message is available from lsh_last_error()
 * (include/lightseq_hip.h).  Device buffers for inputs and outputs are owned by the
 * caller (the model also owns a default set, used until a pointer is set), exactly
 * as in the reference; ls_model_infer() is synchronous.
 *
 * Model classes: "QuantBert" (quant_bert.proto file; input 0 "token_ids" int32
 * [batch, seq_len]; output 0 "encoder_output" fp16 [batch, seq_len, hidden]),
 * pywrapper/quant_bert.cc:6-149.
 */
#ifndef LIGHTSEQ_MODEL_H_
#define LIGHTSEQ_MODEL_H_

#include "lightseq_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ls_model ls_model;

/* values of lightseq::cuda::DataType, model_base.h:12-26 */
enum {
  LS_DTYPE_NOT_SUPPORTED = 0, LS_DTYPE_FLOAT32 = 1, LS_DTYPE_INT32 = 2, LS_DTYPE_INT64 = 3,
  LS_DTYPE_FLOAT16 = 4, LS_DTYPE_INT8 = 5
};
#define LS_MAX_DIMS 8

/* LSModelFactory::GetInstance().CreateModel(class_name, weight_path, max_batch_size),
 * model_base.h:126-135 */
int ls_model_create(const char* class_name, const char* weight_path, int max_batch_size,
                    ls_model** model);
int ls_model_destroy(ls_model* model);
/* LSModel::Infer, model_base.h:69 */
int ls_model_infer(ls_model* model);
/* model_base.h:72-79 */
int ls_model_set_input_ptr(ls_model* model, int index, void* input_ptr);
int ls_model_set_input_shape(ls_model* model, int index, const int* shape, int ndim);
int ls_model_get_input_max_shape(ls_model* model, int index, int* shape /*[LS_MAX_DIMS]*/,
                                 int* ndim);
int ls_model_get_input_size(ls_model* model, int* count);
int ls_model_get_input_name(ls_model* model, int index, const char** name);
int ls_model_get_input_dtype(ls_model* model, int index, int* dtype);
/* model_base.h:82-89 */
int ls_model_set_output_ptr(ls_model* model, int index, void* output_ptr);
int ls_model_get_output_ptr(ls_model* model, int index, const void** output_ptr);
int ls_model_get_output_size(ls_model* model, int* count);
int ls_model_get_output_name(ls_model* model, int index, const char** name);
int ls_model_get_output_shape(ls_model* model, int index, int* shape /*[LS_MAX_DIMS]*/, int* ndim);
int ls_model_get_output_max_shape(ls_model* model, int index, int* shape /*[LS_MAX_DIMS]*/,
                                  int* ndim);
int ls_model_get_output_dtype(ls_model* model, int index, int* dtype);
/* model_base.h:91 */
int ls_model_benchmark_mode(ls_model* model, int is_benchmark);

/* No counterpart in the reference: the HIP stream the model launches on, so that a
 * caller can bracket ls_model_infer() with events on that stream. */
int ls_model_get_stream(ls_model* model, lsh_stream_t* stream);
/* No counterpart in the reference (it times whole Infer() calls on the host): when
 * enabled, a QuantBert model brackets every int8 GEMM launch with HIP events on its
 * stream; ls_model_get_profile() writes a JSON array with, per GEMM site (qkv,
 * attn_out, ffn1, ffn2): kernel instantiation, m, n, k, launches and total_ms
 * accumulated since profiling was switched on.  Enabling resets the counters. */
int ls_model_set_profiling(ls_model* model, int on);
int ls_model_get_profile(ls_model* model, char* buf, int capacity);
/* No counterpart in the reference (its DEBUG_RESULT build prints tensors instead):
 * asks a QuantBert model to copy the named intermediate of encoder layer
 * `layer` into `dst` (device memory, caller-sized) during the next ls_model_infer().
 * Names: ln1_q qkv_q ctx_q out_q ln2_q ffn1_q act_q (int8), ffn2_acc (int32),
 * res_attn res_ffn (fp16 [tokens, hidden]: the residual stream as the LayerNorm kernel
 * after the attention out-projection / after FFN2 reads it).  dst NULL clears. */
int ls_model_set_tap(ls_model* model, int layer, const char* name, void* dst);
/* No counterpart in the reference.  Names that start with "dec." tap one generation step
 * of QuantTransformer's decoder or of QuantGpt instead: the intermediate of decoder layer
 * `layer` at the step given to ls_model_set_tap_step() (QuantTransformer: the decoding step,
 * from 0; QuantGpt: the number of tokens sampled before the cached step, from 1).
 * QuantTransformer (rows = batch * beam): dec.self_ln_q dec.self_q dec.self_ctx_q
 * dec.self_out_q dec.encdec_ln_q dec.encdec_ctx_q dec.encdec_out_q dec.ffn_ln_q
 * dec.next_ln_q (int8 [rows, hidden]), dec.ffn1_act_q (int8 [rows, inner]), dec.ffn2_acc
 * (int32 [rows, hidden]), dec.self_k_cache dec.self_v_cache (int8 [rows, heads, max_step,
 * d], after the step's append), dec.encdec_q (fp16 [batch, heads, beam, d]), dec.encdec_k
 * dec.encdec_v (fp16 [batch, heads, src_len, d]), dec.res_in dec.res_self dec.res_encdec
 * dec.res_out (fp16 [rows, hidden]: the residual stream at the start of the layer and
 * after each of its three layer norms).
 * QuantGpt (rows = batch): dec.ln1_q dec.self_q dec.ctx_q dec.out_q dec.ln2_q
 * dec.next_ln_q (int8 [rows, hidden]), dec.act_q (int8 [rows, inner]), dec.ffn2_acc,
 * dec.k_cache dec.v_cache, dec.res_in dec.res_attn dec.res_out.
 * While any step tap is set the steps are not replayed as graphs. */
int ls_model_set_tap_step(ls_model* model, int step);
/* QuantTransformer only: the tap "enc_out" (layer ignored) receives the encoder output
 * [batch, seq_len, hidden] fp16 of every Infer().
 *
 * Debug aid without counterpart in the reference, QuantTransformer only: record, for the
 * first max_steps decoding steps of every Infer(), the int8 logits [step, batch*beam,
 * vocab] and the sequences after the step [step, batch*beam, max_step] (either may be
 * NULL).  ls_model_get_steps_run gives the number of steps the last Infer() ran. */
int ls_model_set_step_record(ls_model* model, int8_t* logits, int* alive_seq, int max_steps);
int ls_model_get_steps_run(ls_model* model, int* steps);
/* Measurement aid without counterpart in the reference, QuantTransformer and QuantGpt: GPU time
 * of the last Infer() between HIP events on the model's stream -- prepare_ms: before the step
 * loop (QuantTransformer: the K/V projection of the encoder output; QuantGpt: the prompt pass
 * and the first token), steps_ms: the step loop, steps: the steps it ran. */
int ls_model_get_phase_times(ls_model* model, float* prepare_ms, float* steps_ms, int* steps);
/* No counterpart in the reference (its step loops launch kernel by kernel:
 * model/quant_decoder.cc.cu:446-454, quant_gpt_encoder.cc.cu:361-389).  QuantTransformer and
 * QuantGpt: when on, every generation step -- embedding, the layer stack, the logits GEMM, the
 * search / sampling kernels and the cache reorder -- is replayed as one HIP graph.  A step's
 * launches depend only on the shapes of the call and the step's position, so graphs are kept
 * per (batch size, source or prompt length, step): the first call with a key runs eagerly, the
 * second captures, later ones replay.  The early-stop word is read back between replays as
 * before.  Ignored while a step record is set.  Results are identical either way.
 * ls_model_get_graph_stats: graphs captured so far, steps replayed so far. */
int ls_model_set_graph_mode(ls_model* model, int on);
int ls_model_get_graph_stats(ls_model* model, int* captured, long long* replayed);
/* nodes (kernel launches and copies) of the step graph captured last: the launches of one step */
int ls_model_get_graph_nodes(ls_model* model, int* nodes);

/* QuantGpt with sampling_method topk (topk > 1) or topp, QuantTransformer with sampling_method
 * topk or topp (model/quant_decoder.cc.cu:952-998): restart the per-sequence generator
 * states of the sampling steps (sequence i of a batch draws from Philox4x32-10 keyed with `seed`,
 * counter (draw, 0, i, 0)).  A model starts with seed 0, so two runs of one model file give the
 * same tokens; the reference seeds its cuRAND states with clock()
 * (kernels/transformerKernels.cc.cu:2270-2274, model/quant_gpt_encoder.cc.cu:66-71) and defines
 * no stream of numbers.  No counterpart in the reference. */
int ls_model_set_seed(ls_model* model, unsigned long long seed);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTSEQ_MODEL_H_ */
