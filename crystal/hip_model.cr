# Crystal binding of the layer- and model-level entry points of
# libshainet_hip_kernels.so: the whole LlamaBlock, the model walk of Network#run,
# the Sampler's device half and HFLoader.load_llama.  Bound like the rest of the
# kernel library, by dlopen / dlsym (hip.cr: `HIP.sym`, the idiom of cuda.cr:841-852),
# so that a build that never opens the library still links; every function returns
# the Int32 status of the rest of the library (0 = ok, 1 = ArgumentError,
# 3 = allocation failed).
#
# Written without a Crystal compiler at hand (none exists in the build image).
require "./hip"

module SHAInet
  module HIP
    alias Model = Pointer(Void)
    alias Block = Pointer(Void)

    # One cached Proc per entry point: `model_fn(name, arg types..., return type)`.
    macro model_fn(name, *types)
      @@{{name.id}}_proc : Proc({{types.splat}})?

      def self.{{name.id}}(*args)
        fn = (@@{{name.id}}_proc ||= Proc({{types.splat}}).new(HIP.sym({{name.id.stringify}}), Pointer(Void).null))
        fn.call(*args)
      end
    end

    module LibModel
      HIP.model_fn shainet_llama_block_create, Pointer(Block), Int32, Int32, Int32, Float64, Float64, Int32, Int32, Int32
      HIP.model_fn shainet_llama_block_destroy, Block, Int32
      HIP.model_fn shainet_llama_block_attn, Block, Pointer(Void)
      HIP.model_fn shainet_llama_block_set_norms, Block, Pointer(Float32), Pointer(Float32), Int32
      HIP.model_fn shainet_llama_block_set_ffn, Block, Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32
      HIP.model_fn shainet_llama_block_clear_cache, Block, Int32
      HIP.model_fn shainet_llama_block_cache_len, Block, Int32
      HIP.model_fn shainet_llama_block_forward_cached, Block, Pointer(Float32), Int32, Pointer(Float32), Int32, Int32
      HIP.model_fn shainet_llama_block_forward, Block, Pointer(Float32), Int32, Pointer(Float32), Int32, Int32

      HIP.model_fn shainet_llama_attn_set_rope, Pointer(Void), Float64, Pointer(Float32), Int32
      HIP.model_fn shainet_llama_attn_set_qk_norm, Pointer(Void), Pointer(Float32), Int32, Pointer(Float32), Int32, Int32
      HIP.model_fn shainet_llama_attn_set_bias, Pointer(Void), Pointer(Float32), Int32, Pointer(Float32), Int32, Pointer(Float32), Int32, Int32
      HIP.model_fn shainet_llama_attn_set_weights, Pointer(Void), Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32

      HIP.model_fn shainet_llama_model_create, Pointer(Model), Int32, Int32, Int32, Int32, Int32, Int32, Int32, Float64, Float64, Int32
      HIP.model_fn shainet_llama_model_destroy, Model, Int32
      HIP.model_fn shainet_llama_model_block, Model, Int32, Block
      HIP.model_fn shainet_llama_model_set_embedding, Model, Pointer(Float32), Int32
      HIP.model_fn shainet_llama_model_set_final_norm, Model, Pointer(Float32), Int32
      HIP.model_fn shainet_llama_model_set_lm_head, Model, Pointer(Float32), Pointer(Float32), Int32
      HIP.model_fn shainet_llama_model_clear_cache, Model, Int32
      HIP.model_fn shainet_llama_model_run, Model, Pointer(Int32), Int32, Pointer(Float32), Int32
      HIP.model_fn shainet_llama_model_greedy, Model, Pointer(Int32), Int32
      HIP.model_fn shainet_llama_model_repetition_penalty, Model, Pointer(Int32), Int32, Float64, Int32
      HIP.model_fn shainet_llama_model_topk, Model, Int32, Pointer(Int32), Pointer(Float32), Pointer(Int32), Int32
      HIP.model_fn shainet_llama_model_sample, Model, Int32, Float64, Float64, Pointer(Int32), Int32
      HIP.model_fn shainet_llama_model_generate_greedy, Model, Int32, Pointer(Int32), Int32, Pointer(Int32), Pointer(Int32), Int32
      HIP.model_fn shainet_hf_load_llama, Pointer(UInt8), Pointer(Model), Int32
    end

    def self.check!(status : Int32)
      HIP.check(status)
    end

    # Network#run(ids) with use_kv_cache for a network whose LLaMA stack lives on the
    # device (network_run.cr:185-226): returns the [1, vocab] logits row.
    class DeviceLlama
      getter vocab : Int32

      def initialize(@handle : Model, @vocab : Int32)
      end

      # HFLoader.load_llama(model_dir) (hf_loader.cr:277-412), dense models
      def self.load(model_dir : String, vocab : Int32) : DeviceLlama
        h = Model.null
        HIP.check!(LibModel.shainet_hf_load_llama(model_dir.to_unsafe, pointerof(h)))
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

      # Sampler#sample (text/sampler.cr:88-150) on the device logits: top-k, temperature softmax
      # over the survivors and the inverse-CDF pick for the uniform draw `r` in [0, 1) that the
      # caller's random generator made.
      def sample(top_k : Int32, temperature : Float64, r : Float64) : Int32
        id = 0
        HIP.check!(LibModel.shainet_llama_model_sample(@handle, top_k, temperature, r, pointerof(id)))
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
