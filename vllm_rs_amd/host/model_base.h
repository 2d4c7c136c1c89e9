// model_base.h — what the engine asks of a model: weights in, a paged cache, one forward per step.  The engine (engine.cpp) picks
// the class from vra_model_config.arch (make_model): the Llama / Qwen family (model.h) or a config-driven layer stack (stack_model.h).
#pragma once
#include <stdint.h>

#include <memory>
#include <string>

#include "../../include/vllm_rs_amd.h"

namespace vra {

// The data contract between runner and kernels (InputMetadata, runner.rs:1222-1238,1369-1385);
// all pointers are device buffers owned by the runner.
struct InputMetadata {
  bool is_prefill = false;
  int n_tokens = 0;
  int n_seqs = 0;
  const uint32_t* input_ids = nullptr;      // [T]
  const int64_t* positions = nullptr;       // [T]
  const int64_t* slot_mapping = nullptr;    // [T]
  const uint32_t* block_tables = nullptr;   // [B, max_blocks]
  const uint32_t* context_lens = nullptr;   // [B]
  const uint32_t* cu_seqlens_q = nullptr;   // [B+1] (prefill)
  const uint32_t* last_token_rows = nullptr;  // [B] = seqlens[i]-1 (llama.rs:306-310)
  int max_blocks = 0;
  int max_seqlen_q = 0;
  int max_context_len = 0;
  // rows of the step whose logits are wanted, in order (replayed traces ask for several per sequence); 0: the last row of every
  // sequence of a prefill step, every row of a decode step
  const uint32_t* logit_rows = nullptr;  // [n_logit_rows]
  int n_logit_rows = 0;
  // slot of every sequence's recurrent state (models with state_bytes_per_slot() > 0); -1: a padded lane, nothing read or written.
  // A sequence whose first token of the step stands at position 0 starts from a zero state whatever its slot holds.
  const int32_t* state_slots = nullptr;  // [B]
  // the token before each sequence's first row of the step (models that embed token pairs); unused at position 0
  const uint32_t* prev_tokens = nullptr;  // [B]
};

class ModelBase {
 public:
  virtual ~ModelBase() {}
  std::string error;
  // weights
  virtual bool init_synthetic(uint64_t seed) = 0;
  virtual bool load_tensor(const std::string& name, const void* host, const int64_t* shape, int ndim, int elem_bytes) = 0;
  virtual bool finalize_weights() = 0;
  // paged cache: `kv_layers()` layers own one; a block of layer l is k_block_bytes(l) / v_block_bytes(l) contiguous bytes
  virtual bool init_kv_cache(int num_blocks) = 0;
  virtual int num_blocks() const = 0;
  virtual int kv_layers() const = 0;
  virtual size_t k_block_bytes(int l) const = 0;
  virtual size_t v_block_bytes(int l) const = 0;
  virtual void* k_cache(int l) const = 0;
  virtual void* v_cache(int l) const = 0;
  // bytes of ONE block over all layers, K and V (the engine plans the block count from free memory with it)
  virtual int64_t kv_bytes_per_block() const = 0;
  // what the model carries from token to token for ONE sequence beside the paged cache, in bytes (0: nothing); the engine hands out
  // `slots` slots through its block manager (core.h StateSlots) and names each sequence's slot in InputMetadata::state_slots
  virtual int64_t state_bytes_per_slot() const { return 0; }
  virtual bool init_state(int /*slots*/) { return true; }
  virtual bool init_buffers(int max_tokens, int max_seqs) = 0;
  // rows of logits one forward can leave (>= max_seqs)
  virtual int max_logit_rows() const = 0;
  virtual void set_comm(void* comm) = 0;
  virtual bool has_comm() const = 0;
  virtual int world() const = 0;
  // forward -> f32 logits [rows, vocab] on the device; tokens != null: the greedy token of every logits row as well
  virtual bool forward(const InputMetadata& md, int64_t stream, uint32_t* tokens = nullptr) = 0;
  virtual float* logits() const = 0;
  virtual size_t weight_bytes() const = 0;
  // decode steps may be captured into hipGraphs at init
  virtual bool graph_capturable() const { return true; }
  // instrumentation of the Llama family (model.h); other models answer "nothing"
  virtual bool launch_gemm(int, int, int, int64_t) { return false; }
  virtual int64_t gemm_algorithmic_bytes(int, int) const { return 0; }
  virtual int norm_deferred_mask(int, int = 1) const { return 0; }
  virtual void set_tp_snapshots(int) {}
  virtual int64_t read_tp_snapshot(int, void*, int64_t, int64_t) { return -1; }
  // the residual stream after every layer run of the LAST forward, f32 [layer runs, rows, width]: parity instrumentation of layer
  // stacks (off by default: no buffers, no copies); -1 = not offered
  virtual void set_layer_trace(bool) {}
  virtual int64_t read_layer_trace(void*, int64_t, int64_t) { return -1; }
};

// `spec`: the layer list of a layer-stack model (stack_model.h), null for the Llama family
std::unique_ptr<ModelBase> make_model(const vra_model_config& mc, const vra_engine_config& ec, const char* spec, std::string* error);

}  // namespace vra
