# Crystal binding of the layer- and model-level entry points of
# libshainet_hip_kernels.so: the whole LlamaBlock, the model walk of Network#run,
# the Sampler's device half and HFLoader.load_llama.  The library is linked
# directly (`@[Link]`), the way the reference links its runtime library
# (cuda.cr:9-19); every function returns the Int32 status of the rest of the
# library (0 = ok, 1 = ArgumentError, 3 = allocation failed).
#
# Written without a Crystal compiler at hand (none exists in the build image).
require "./hip"

module SHAInet
  module HIP
    @[Link("shainet_hip_kernels")]
    lib LibModel
      type Attn = Void*
      type Block = Void*
      type Model = Void*

      fun shainet_hip_last_error : LibC::Char*

      fun shainet_llama_block_create(out : Block*, d_model : Int32, num_heads : Int32, ff_hidden : Int32, eps : Float64,
                                     rope_theta : Float64, num_kv_heads : Int32, head_dim : Int32) : Int32
      fun shainet_llama_block_destroy(block : Block) : Int32
      fun shainet_llama_block_attn(block : Block) : Attn
      fun shainet_llama_block_set_norms(block : Block, norm1 : Float32*, norm2 : Float32*) : Int32
      fun shainet_llama_block_set_ffn(block : Block, gate : Float32*, up : Float32*, down : Float32*) : Int32
      fun shainet_llama_block_clear_cache(block : Block) : Int32
      fun shainet_llama_block_cache_len(block : Block) : Int32
      fun shainet_llama_block_forward_cached(block : Block, x : Float32*, new_tokens : Int32, out : Float32*, mem : Int32) : Int32

      fun shainet_llama_attn_set_rope(attn : Attn, rope_theta : Float64, rope_freqs : Float32*) : Int32
      fun shainet_llama_attn_set_qk_norm(attn : Attn, q_norm : Float32*, q_len : Int32, k_norm : Float32*, k_len : Int32) : Int32
      fun shainet_llama_attn_set_bias(attn : Attn, b_q : Float32*, q_len : Int32, b_k : Float32*, k_len : Int32,
                                      b_v : Float32*, v_len : Int32) : Int32
      fun shainet_llama_attn_set_weights(attn : Attn, w_q : Float32*, w_k : Float32*, w_v : Float32*, w_o : Float32*) : Int32

      fun shainet_llama_model_create(out : Model*, vocab : Int32, d_model : Int32, n_layers : Int32, num_heads : Int32,
                                     num_kv_heads : Int32, head_dim : Int32, ff_hidden : Int32, eps : Float64,
                                     rope_theta : Float64) : Int32
      fun shainet_llama_model_destroy(model : Model) : Int32
      fun shainet_llama_model_block(model : Model, layer : Int32) : Block
      fun shainet_llama_model_set_embedding(model : Model, table : Float32*) : Int32
      fun shainet_llama_model_set_final_norm(model : Model, gamma : Float32*) : Int32
      fun shainet_llama_model_set_lm_head(model : Model, weights : Float32*, bias : Float32*) : Int32
      fun shainet_llama_model_clear_cache(model : Model) : Int32
      fun shainet_llama_model_run(model : Model, tokens : Int32*, n_tokens : Int32, logits : Float32*) : Int32
      fun shainet_llama_model_greedy(model : Model, token : Int32*) : Int32
      fun shainet_llama_model_repetition_penalty(model : Model, recent_ids : Int32*, n : Int32, penalty : Float64) : Int32
      fun shainet_llama_model_topk(model : Model, k : Int32, ids : Int32*, vals : Float32*, count : Int32*) : Int32
      fun shainet_llama_model_generate_greedy(model : Model, max_tokens : Int32, stop_ids : Int32*, n_stop : Int32,
                                              out : Int32*, n_out : Int32*) : Int32
      fun shainet_hf_load_llama(model_dir : LibC::Char*, out : Model*) : Int32
    end

    def self.check!(status : Int32)
      return if status == 0
      msg = String.new(LibModel.shainet_hip_last_error)
      raise ArgumentError.new(msg) if status == 1
      raise msg
    end

    # Network#run(ids) with use_kv_cache for a network whose LLaMA stack lives on the
    # device (network_run.cr:185-226): returns the [1, vocab] logits row.
    class DeviceLlama
      getter vocab : Int32

      def initialize(@handle : LibModel::Model, @vocab : Int32)
      end

      # HFLoader.load_llama(model_dir) (hf_loader.cr:277-412), dense models
      def self.load(model_dir : String, vocab : Int32) : DeviceLlama
        h = Pointer(Void).null.as(LibModel::Model)
        HIP.check!(LibModel.shainet_hf_load_llama(model_dir, pointerof(h)))
        new(h, vocab)
      end

      def run(ids : Array(Int32)) : SimpleMatrix
        logits = SimpleMatrix.new(1, @vocab)
        HIP.check!(LibModel.shainet_llama_model_run(@handle, ids.to_unsafe, ids.size, logits.data.to_unsafe))
        logits
      end

      def clear_cache!
        HIP.check!(LibModel.shainet_llama_model_clear_cache(@handle))
      end

      # Sampler.greedy on the logits the last run left on the device
      def greedy : Int32
        id = 0
        HIP.check!(LibModel.shainet_llama_model_greedy(@handle, pointerof(id)))
        id
      end

      # The loop of examples/llama_chat.cr:181-197 with greedy selection
      def generate_greedy(max_tokens : Int32, stop_ids : Array(Int32)) : Array(Int32)
        out = Array(Int32).new(max_tokens, 0)
        n = 0
        HIP.check!(LibModel.shainet_llama_model_generate_greedy(@handle, max_tokens, stop_ids.to_unsafe, stop_ids.size,
          out.to_unsafe, pointerof(n)))
        out[0, n]
      end

      def finalize
        LibModel.shainet_llama_model_destroy(@handle)
      end
    end
  end
end
