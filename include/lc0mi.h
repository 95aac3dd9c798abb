/*
 * lc0mi -- C ABI of the MI355X (gfx950) neural-network backend for lc0.
 *
 * Every entry point replaces one member of lc0's backend interface
 * (reference file:line given per function). No C++ types or exceptions cross
 * this boundary: functions return 0 on success and a non-zero code on failure,
 * and lc0mi_last_error() then holds the message lc0 would have received as
 * lczero::Exception (src/utils/exception.h:36-41). The library has no CPU
 * fallback: creating a network without a HIP device fails.
 *
 * Threading: a lc0mi_net may be shared by any number of threads; a lc0mi_comp
 * belongs to one thread at a time (src/neural/network.h:56-71 contract).
 */
#ifndef LC0MI_H_
#define LC0MI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct lc0mi_net lc0mi_net;   /* device weights + buffer pool */
typedef struct lc0mi_comp lc0mi_comp; /* one batch in flight */

/* Factory, replaces MakeBlasNetwork/REGISTER_NETWORK factories
 * (src/neural/backends/blas/network_blas.cc:1115-1187, src/neural/factory.h:111-142).
 * `data` is a serialized pblczero.Net (raw, or gzip-compressed): what
 * WeightsFile::OutputAsString() yields (src/utils/protomessage.h:29).
 * `opts_kv` is "key=value,key=value": gpu=<id>, max_batch=<n>, precision=fp16,
 * policy_head=<name>, value_head=<name>, mlh=<bool>; unknown keys are errors
 * (src/neural/wrapper.cc:194). May be NULL. */
int lc0mi_net_create_from_buffer(const void* data, size_t len, const char* opts_kv, lc0mi_net** out);
/* Same from a .pb.gz file, replaces LoadWeightsFromFile + factory
 * (src/neural/loader.cc:190-212). */
int lc0mi_net_create_from_file(const char* pb_gz_path, const char* opts_kv, lc0mi_net** out);
/* Replaces ~Network (src/neural/network.h:118). */
void lc0mi_net_destroy(lc0mi_net* net);
/* Replaces Network::GetCapabilities (src/neural/network.h:119): the three enum
 * values of pblczero.NetworkFormat input / output / moves_left. */
int lc0mi_net_caps(const lc0mi_net* net, int* input_format, int* output_format, int* moves_left_format);
/* Replaces Network::GetMiniBatchSize / GetPreferredBatchStep / GetThreads /
 * IsCpu (src/neural/network.h:121-125) plus the largest batch one device pass takes. */
int lc0mi_net_hints(const lc0mi_net* net, int* minibatch, int* batch_step, int* max_batch, int* threads,
                    int* is_cpu);

/* Replaces Network::NewComputation (src/neural/network.h:120). */
int lc0mi_comp_create(lc0mi_net* net, lc0mi_comp** out);
/* Replaces ~NetworkComputation; returns the pinned buffers to the pool. */
void lc0mi_comp_destroy(lc0mi_comp* comp);
/* Replaces NetworkComputation::AddInput (src/neural/network.h:59): one position
 * = 112 InputPlane{mask,value} (src/neural/network.h:43-52), split in two arrays. */
int lc0mi_comp_add_input(lc0mi_comp* comp, const uint64_t masks[112], const float values[112]);
/* n positions at once (masks[n][112], values[n][112]). */
int lc0mi_comp_add_inputs(lc0mi_comp* comp, int n, const uint64_t* masks, const float* values);
/* Replaces NetworkComputation::ComputeBlocking (src/neural/network.h:61). */
int lc0mi_comp_compute_blocking(lc0mi_comp* comp);
/* Replaces NetworkComputation::GetBatchSize (src/neural/network.h:63). */
int lc0mi_comp_batch_size(const lc0mi_comp* comp);
/* Replace GetQVal / GetDVal / GetMVal / GetPVal (src/neural/network.h:65-70):
 * q = W-L after softmax (or tanh value), d = draw probability or 0, m = moves
 * left (ReLU) or 0, p = RAW policy logit of move_id in [0,1858). On a bad index
 * or before compute they return NaN and set the error string. */
float lc0mi_comp_q(const lc0mi_comp* comp, int sample);
float lc0mi_comp_d(const lc0mi_comp* comp, int sample);
float lc0mi_comp_m(const lc0mi_comp* comp, int sample);
float lc0mi_comp_p(const lc0mi_comp* comp, int sample, int move_id);
/* All 1858 raw logits of one sample (host memory owned by the computation,
 * valid until it is destroyed); NULL on error. Bulk form of GetPVal. */
const float* lc0mi_comp_policy_row(const lc0mi_comp* comp, int sample);

/* ---- legal-move policy on the device ----
 * Replaces NetworkAsBackendComputation::SoftmaxPolicy (src/neural/wrapper.cc:135-156): the search wrapper
 * fetches the logit of every legal move with GetPVal, subtracts the maximum, multiplies by 1 / temperature,
 * applies FastExp (src/utils/fastmath.h:59-86) and normalises. Given the policy indices of the legal moves
 * (MoveToNNIndex, src/neural/encoder.cc:339-619) the same arithmetic runs on the GPU and only those
 * probabilities are copied to the host, not the 1858 logits.
 *
 * lc0mi_comp_add_legal_moves lists the moves of the input added last (n in 0..256, ids < 1858). Once used it
 * must be called for every input of the computation, right after the input; lc0mi_comp_p and
 * lc0mi_comp_policy_row then fail (the logits stay on the device). */
int lc0mi_comp_add_legal_moves(lc0mi_comp* comp, int n, const uint16_t* move_ids);
/* lc0's PolicyTemperature (src/neural/shared_params.cc:33-36,69); default 1.359. */
int lc0mi_comp_set_policy_softmax_temperature(lc0mi_comp* comp, float temperature);
/* Probabilities of the listed moves of one sample in the order they were listed (host memory owned by the
 * computation); *n receives their number. NULL on error. */
const float* lc0mi_comp_legal_policy(const lc0mi_comp* comp, int sample, int* n);

/* Message of the last failed call on this thread (never NULL). */
const char* lc0mi_last_error(void);

/* ---- measurement hooks (the role of DEBUG_RAW_NPS in
 * src/neural/backends/cuda/network_cuda.cc:715 and of `lc0 backendbench`) ---- */
/* Turns per-kernel HIP-event timing of subsequent compute calls on or off. */
int lc0mi_net_set_profiling(lc0mi_net* net, int on);
/* Writes the accumulated per-kernel records as text lines
 * "name ms launches flops bytes\n" into buf (truncated to cap, NUL-terminated),
 * clears them and returns the number of bytes needed. */
int lc0mi_net_take_profile(lc0mi_net* net, char* buf, int cap);
/* Re-runs the device pass for `batch` positions already resident in HBM `iters`
 * times; *ms_per_pass receives the mean HIP-event time. */
int lc0mi_net_time_resident_forward(lc0mi_net* net, int batch, int iters, double* ms_per_pass);

/* ---- fp8 configuration (backend option precision=fp8, attention-body nets) ----
 * The four large GEMMs of every encoder layer (and by default the smolgen chain, option fp8_gemms) run on e4m3
 * operands: weights with one scale per output row (absmax / 448), activations with one scale per tensor taken from a
 * calibration pass
 * (the reference reaches fp8 only by handing the whole graph to MIGraphX,
 * src/neural/backends/onnx/network_onnx.cc:757, and converts with src/utils/fp8_utils.h:111-155). At creation the network calibrates
 * itself on built-in pseudo-positions; this call replaces those scales with ones derived from n
 * caller-supplied positions (same packed planes as lc0mi_comp_add_inputs). */
int lc0mi_net_calibrate_fp8(lc0mi_net* net, int n, const uint64_t* masks, const float* values);
/* The activation scales in use (value = code x scale), seven floats per encoder layer: the operands of the Q/K/V,
 * attention-output, FFN1 and FFN2 layers, then of smolgen's first dense layer, second dense layer and generator
 * (1 where an operand stays in fp16). Writes at most cap floats and returns the number there are, -1 on error.
 * No counterpart in the reference (it has no fp8 arithmetic of its own); used to check the fp8 pass against an
 * emulation of the same arithmetic. */
int lc0mi_net_fp8_scales(const lc0mi_net* net, float* out, int cap);

/* ---- decoded weights (host only, needs no GPU) ----
 * What the library reads from a weights file, for checking the loader: LayerAdapter decoding of the four
 * Layer encodings (src/utils/weights_adapter.cc:38-62), the batch-norm fold of ConvBlock
 * (src/neural/network_legacy.cc:62-131), the head resolution of MultiHeadWeights (:236-306) and the format
 * upgrades of FixOlderWeightsFile (src/neural/loader.cc:108-158).
 * lc0mi_weights_list writes "format key=value ..." and one "name count" line per non-empty tensor into buf
 * (NUL-terminated, truncated to cap) and returns the bytes needed, -1 on error. */
int lc0mi_weights_list(const void* data, size_t len, char* buf, int cap);
/* Copies tensor `name` (as listed) into out (at most cap floats); returns its element count, -1 on error. */
long long lc0mi_weights_tensor(const void* data, size_t len, const char* name, float* out, long long cap);

/* ---- tables (closed forms of the tables under src/neural/tables, exposed for checking) ---- */
/* kAttnPolicyMap (4288 entries), kConvPolicyMap (4672), kPosEncoding (64*64). */
const int16_t* lc0mi_attn_policy_map(int* count);
const int16_t* lc0mi_conv_policy_map(int* count);
const float* lc0mi_pos_encoding(int* count);

#ifdef __cplusplus
}
#endif
#endif /* LC0MI_H_ */
