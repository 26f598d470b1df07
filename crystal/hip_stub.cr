# Test double used when SHAInet is compiled without -Denable_hip: same module,
# method and class names as hip.cr and hip_model.cr, nothing available, every call
# that would reach the device raises.  The twin of src/shainet/cuda_stub.cr
# (26-28, 97-103) for this path: a CPU-only build compiles and links without
# libamdhip64 and without the kernel library.
module SHAInet
  module HIP
    extend self
    Log = ::Log.for(self)

    enum MemcpyKind
      HostToHost     = 0
      HostToDevice   = 1
      DeviceToHost   = 2
      DeviceToDevice = 3
    end

    MEM_HOST   = 0
    MEM_DEVICE = 1

    alias Handle = Pointer(Void)
    alias Model = Pointer(Void)
    alias Block = Pointer(Void)

    def available? : Bool
      false
    end

    def kernels_available? : Bool
      false
    end

    def fully_available? : Bool
      false
    end

    def last_error : String
      "HIP disabled"
    end

    def free(*args)
    end

    def device_synchronize
    end

    def attn_destroy(*args)
    end

    def kv_cache_destroy(*args)
    end

    {% for name in %w(sym malloc memcpy kv_cache_append_f32 attention_kv_f32 attn_create attn_set_bias
                     kv_cache_create kv_cache_clear kv_cache_len kv_cache_capacity kv_cache_reserve
                     attn_forward attn_forward_noalloc attn_decode_step kv_cache_lengths_to_device
                     kv_cache_lengths_from_device attn_sync rope_apply matmul_f32 check) %}
      def {{name.id}}(*args)
        raise "HIP disabled"
      end
    {% end %}

    def self.check!(status : Int32)
      raise "HIP disabled"
    end

    # hip_model.cr: the entry points behind LibModel are never resolved in this build
    module LibModel
      {% for name in %w(shainet_llama_block_create shainet_llama_block_destroy shainet_llama_block_attn
                       shainet_llama_block_set_norms shainet_llama_block_set_ffn shainet_llama_block_clear_cache
                       shainet_llama_block_cache_len shainet_llama_block_forward_cached shainet_llama_block_forward
                       shainet_llama_attn_set_rope shainet_llama_attn_set_qk_norm shainet_llama_attn_set_bias
                       shainet_llama_attn_set_weights shainet_llama_model_create shainet_llama_model_destroy
                       shainet_llama_model_block shainet_llama_model_set_embedding shainet_llama_model_set_final_norm
                       shainet_llama_model_set_lm_head shainet_llama_model_clear_cache shainet_llama_model_run
                       shainet_llama_model_greedy shainet_llama_model_repetition_penalty shainet_llama_model_topk
                       shainet_llama_model_sample shainet_llama_model_generate_greedy shainet_hf_load_llama) %}
        def self.{{name.id}}(*args)
          raise "HIP disabled"
        end
      {% end %}
    end

    class DeviceLlama
      getter vocab : Int32

      def initialize(@handle : Model, @vocab : Int32)
      end

      def self.load(model_dir : String, vocab : Int32) : DeviceLlama
        raise "HIP disabled"
      end

      {% for name in %w(run clear_cache! greedy sample generate_greedy) %}
        def {{name.id}}(*args)
          raise "HIP disabled"
        end
      {% end %}
    end
  end
end
