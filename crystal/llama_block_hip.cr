# The changes a SHAInet maintainer makes to src/shainet/transformer/llama_block.cr
# so that LlamaBlock#forward_cached runs its attention on an MI355X.  Everything
# else in the class (constructor, properties, forward, clear_cache!, the CPU
# paths) stays as it is.  Written as a reopening of the class so it can be
# required after the original file:
#
#   {% if flag?(:enable_hip) %}
#     require "./hip"            # crystal/hip.cr
#   {% else %}
#     require "./hip_stub"       # crystal/hip_stub.cr
#   {% end %}
#   require "./transformer/llama_block"
#   require "./llama_block_hip"  # this file
#
# attention_cached_cpu (llama_block.cr:246-299) keeps its projections and its
# output projection; the part between them (bias, QK-norm, K RoPE + append, the
# head loop: lines 256-296) becomes ONE library call.  The device cache is the
# cache of record, so the host arrays @k_cache/@v_cache are no longer filled on
# this path and @cache_len mirrors the library's length.
module SHAInet
  class LlamaBlock
    @hip_ctx : HIP::Handle = HIP::Handle.null
    @hip_cache : HIP::Handle = HIP::Handle.null
    @hip_avail : Bool?
    INITIAL_CAPACITY = 256 # llama_block.cr:500

    # llama_block.cr:484-492 with the HIP probes.
    private def hip_attention? : Bool
      return false if force_cpu_attention?
      avail = @hip_avail
      if avail.nil?
        avail = !ENV["SHAINET_CPU_ATTENTION"]? && HIP.fully_available?
        @hip_avail = avail
      end
      avail
    end

    # Parameters are read when the first cached call arrives: HFLoader sets
    # rope_theta, rope_freqs, biases and q/k_norm after construction
    # (hf_loader.cr:319-373).
    private def hip_context : HIP::Handle
      if @hip_ctx.null?
        @hip_ctx = HIP.attn_create(@num_heads, @num_kv_heads, @head_dim, @rope_theta, @rope_freqs,
          @q_norm, @k_norm, @qk_norm_eps, INITIAL_CAPACITY)
        HIP.attn_set_bias(@hip_ctx, @b_q, @b_k, @b_v)
        @hip_cache = HIP.kv_cache_create(@hip_ctx, 1, INITIAL_CAPACITY)
      end
      @hip_ctx
    end

    # Replaces lines 256-296 of attention_cached_cpu when hip_attention? holds.
    # q_full, k_new, v_new are the projection outputs (llama_block.cr:253-255).
    private def attention_cached_hip(q_full : SimpleMatrix, k_new : SimpleMatrix, v_new : SimpleMatrix,
                                     output : SimpleMatrix, new_tokens : Int32)
      ctx = hip_context
      total_len = @cache_len + new_tokens
      cap = HIP.kv_cache_capacity(@hip_cache)
      if total_len > cap # ensure_gpu_cache! (llama_block.cr:497-520): grow by doubling, contents kept on the device
        HIP.kv_cache_reserve(@hip_cache, Math.max(total_len, cap * 2))
      end
      HIP.attn_forward(ctx, @hip_cache, new_tokens, q_full.data.to_unsafe, k_new.data.to_unsafe,
        v_new.data.to_unsafe, output.data.to_unsafe)
      @cache_len = total_len
    end

    # In attention_cached_cpu, after the three projections:
    #
    #   output = SimpleMatrix.new(new_tokens, @q_dim)
    #   if hip_attention?
    #     attention_cached_hip(q_full, k_new, v_new, output, new_tokens)
    #     return gpu_matmul(output, @w_o)
    #   end
    #   ... the existing lines 256-298 ...

    # clear_cache! (llama_block.cr:116-122) additionally resets the device lengths.
    def clear_cache!
      previous_def
      HIP.kv_cache_clear(@hip_cache) unless @hip_cache.null?
    end

    # finalize (llama_block.cr:124-130) additionally releases the library's handles.
    def finalize
      previous_def
      HIP.kv_cache_destroy(@hip_cache) unless @hip_cache.null?
      HIP.attn_destroy(@hip_ctx) unless @hip_ctx.null?
    end
  end
end
