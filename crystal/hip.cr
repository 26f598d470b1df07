# Crystal binding of libshainet_hip_kernels.so for the LlamaBlock attention path.
#
# Takes the place of src/shainet/cuda.cr for this path only (cuda.cr:9-19, 47-52,
# 124-156, 281, 308-309, 778-780, 834-891): the runtime library is linked
# (`@[Link("amdhip64")]`), the kernel library is opened with dlopen/dlsym and its
# entry points are cached as Procs, exactly as the reference does for
# libshainet_cuda_kernels.so.  Compile with -Denable_hip; without the flag
# hip_stub.cr provides the same module with `fully_available? == false`.
#
# This file was written without a Crystal compiler at hand (none exists in the
# build image); it follows the reference's own binding idioms line for line.
require "log"

module SHAInet
  module HIP
    Log = ::Log.for(self)
    extend self

    KERNEL_LIB = "libshainet_hip_kernels.so"

    @[Link("amdhip64")]
    lib LibHIPRuntime
      fun hipRuntimeGetVersion(version : Pointer(Int32)) : Int32
      fun hipMalloc(ptr : Pointer(Pointer(Void)), size : LibC::SizeT) : Int32
      fun hipFree(ptr : Pointer(Void)) : Int32
      fun hipMemcpy(dst : Pointer(Void), src : Pointer(Void), count : LibC::SizeT, kind : Int32) : Int32
      fun hipMemGetInfo(free : Pointer(LibC::SizeT), total : Pointer(LibC::SizeT)) : Int32
      fun hipDeviceSynchronize : Int32
    end

    # Same numeric values as cudaMemcpyKind (cuda.cr:47-52).
    enum MemcpyKind
      HostToHost     = 0
      HostToDevice   = 1
      DeviceToHost   = 2
      DeviceToDevice = 3
    end

    MEM_HOST   = 0
    MEM_DEVICE = 1

    @@checked = false
    @@available = false
    @@kernels_handle : Pointer(Void) = Pointer(Void).null

    private def kernels_handle : Pointer(Void)
      if @@kernels_handle.null?
        @@kernels_handle = LibC.dlopen(KERNEL_LIB, LibC::RTLD_LAZY)
      end
      @@kernels_handle
    end

    # Address of an entry point of the kernel library (also used by hip_model.cr).
    def sym(name : String) : Pointer(Void)
      h = kernels_handle
      raise "HIP kernels not available" if h.null?
      s = LibC.dlsym(h, name)
      raise "HIP kernels not available" if s.null?
      s
    end

    # cuda.cr:63-83: can the runtime be opened?  SHAINET_DISABLE_HIP short-circuits.
    def available?
      return false if ENV["SHAINET_DISABLE_HIP"]?
      return @@available if @@checked
      @@checked = true
      rt = LibC.dlopen("libamdhip64.so", LibC::RTLD_LAZY)
      @@available = !rt.null?
      LibC.dlclose(rt) unless rt.null?
      @@available
    rescue ex
      Log.error { "HIP availability check raised: #{ex}" }
      @@available = false
    end

    # cuda.cr:111-122, plus the library's own probe for a gfx950 device.
    def kernels_available?
      return false if kernels_handle.null?
      fn = Proc(Int32).new(sym("shainet_hip_available"), Pointer(Void).null)
      fn.call == 1
    rescue ex
      Log.error { "kernel availability check raised: #{ex}" }
      false
    end

    # cuda.cr:778-780
    def fully_available?
      available? && kernels_available?
    end

    def last_error : String
      fn = Proc(Pointer(UInt8)).new(sym("shainet_hip_last_error"), Pointer(Void).null)
      String.new(fn.call)
    end

    # cuda.cr:124-140: a failed allocation may only mean that finalizers have not
    # run yet; collect once and retry before giving up.
    def malloc(ptr : Pointer(Pointer(Void)), size : LibC::SizeT)
      rslt = LibHIPRuntime.hipMalloc(ptr, size)
      unless rslt.zero?
        GC.collect
        rslt = LibHIPRuntime.hipMalloc(ptr, size)
      end
      unless rslt.zero?
        Log.error { "HIP.malloc: hipMalloc failed with result #{rslt} for size #{size}" }
        raise "HIP memory allocation failed"
      end
      rslt
    end

    def free(ptr : Pointer(Void))
      LibHIPRuntime.hipFree(ptr)
    end

    def memcpy(dst : Pointer(Void), src : Pointer(Void), bytes : LibC::SizeT, kind : MemcpyKind)
      LibHIPRuntime.hipMemcpy(dst, src, bytes, kind.value)
    end

    def device_synchronize
      LibHIPRuntime.hipDeviceSynchronize
    end

    # ---- the two entry points with the reference's names (cuda.cr:838-891) ----
    @@kv_cache_append_f32_proc : Proc(Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Int32, Int32, Void)?
    @@attention_kv_f32_proc : Proc(Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Int32, Int32, Int32, Float32, Void)?

    def kv_cache_append_f32(staging : Pointer(Float32), kc : Pointer(Float32), vc : Pointer(Float32),
                            new_tokens : Int32, start_pos : Int32, num_kv_heads : Int32,
                            head_dim : Int32, capacity : Int32)
      fn = (@@kv_cache_append_f32_proc ||= Proc(Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Int32, Int32, Void).new(sym("kv_cache_append_f32"), Pointer(Void).null))
      fn.call(staging, kc, vc, new_tokens, start_pos, num_kv_heads, head_dim, capacity)
    end

    def attention_kv_f32(q : Pointer(Float32), kc : Pointer(Float32), vc : Pointer(Float32),
                         out_ptr : Pointer(Float32), ws : Pointer(Float32),
                         new_tokens : Int32, start_pos : Int32, num_heads : Int32,
                         heads_per_kv : Int32, head_dim : Int32, capacity : Int32, scale : Float32)
      fn = (@@attention_kv_f32_proc ||= Proc(Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Int32, Int32, Int32, Float32, Void).new(sym("attention_kv_f32"), Pointer(Void).null))
      fn.call(q, kc, vc, out_ptr, ws, new_tokens, start_pos, num_heads, heads_per_kv, head_dim, capacity, scale)
    end

    # ---- fused entry points (include/shainet_hip_attn.h) ----------------------
    alias Handle = Pointer(Void)

    def check(status : Int32)
      return if status == 0
      msg = last_error
      raise ArgumentError.new(msg) if status == 1
      if status == 3 # allocation: finalizers may free device memory (cuda.cr:124-140)
        raise "HIP memory allocation failed: #{msg}"
      end
      raise "HIP attention call failed (#{status}): #{msg}"
    end

    def attn_create(num_heads : Int32, num_kv_heads : Int32, head_dim : Int32, rope_theta : Float64,
                    rope_freqs : Array(Float32)?, q_norm : Array(Float32)?, k_norm : Array(Float32)?,
                    eps : Float64, max_positions : Int32) : Handle
      fn = Proc(Pointer(Handle), Int32, Int32, Int32, Float64, Pointer(Float32), Pointer(Float32), Int32, Pointer(Float32), Int32, Float64, Int32, Int32).new(sym("shainet_attn_create"), Pointer(Void).null)
      h = Handle.null
      nullf = Pointer(Float32).null
      args = {rope_freqs ? rope_freqs.to_unsafe : nullf,
              q_norm ? q_norm.to_unsafe : nullf, q_norm ? q_norm.size : -1,
              k_norm ? k_norm.to_unsafe : nullf, k_norm ? k_norm.size : -1}
      status = fn.call(pointerof(h), num_heads, num_kv_heads, head_dim, rope_theta, args[0], args[1], args[2], args[3], args[4], eps, max_positions)
      if status == 3
        GC.collect
        status = fn.call(pointerof(h), num_heads, num_kv_heads, head_dim, rope_theta, args[0], args[1], args[2], args[3], args[4], eps, max_positions)
      end
      check(status)
      h
    end

    def attn_set_bias(ctx : Handle, b_q : Array(Float32)?, b_k : Array(Float32)?, b_v : Array(Float32)?)
      fn = Proc(Handle, Pointer(Float32), Int32, Pointer(Float32), Int32, Pointer(Float32), Int32, Int32).new(sym("shainet_attn_set_bias"), Pointer(Void).null)
      nullf = Pointer(Float32).null
      check fn.call(ctx, b_q ? b_q.to_unsafe : nullf, b_q ? b_q.size : -1,
        b_k ? b_k.to_unsafe : nullf, b_k ? b_k.size : -1,
        b_v ? b_v.to_unsafe : nullf, b_v ? b_v.size : -1)
    end

    def attn_destroy(ctx : Handle)
      Proc(Handle, Int32).new(sym("shainet_attn_destroy"), Pointer(Void).null).call(ctx)
    end

    def kv_cache_create(ctx : Handle, batch : Int32, capacity : Int32) : Handle
      fn = Proc(Pointer(Handle), Handle, Int32, Int32, Int32).new(sym("shainet_kv_cache_create"), Pointer(Void).null)
      h = Handle.null
      status = fn.call(pointerof(h), ctx, batch, capacity)
      if status == 3
        GC.collect
        status = fn.call(pointerof(h), ctx, batch, capacity)
      end
      check(status)
      h
    end

    def kv_cache_destroy(cache : Handle)
      Proc(Handle, Int32).new(sym("shainet_kv_cache_destroy"), Pointer(Void).null).call(cache)
    end

    def kv_cache_clear(cache : Handle, seq : Int32 = -1)
      check Proc(Handle, Int32, Int32).new(sym("shainet_kv_cache_clear"), Pointer(Void).null).call(cache, seq)
    end

    def kv_cache_len(cache : Handle, seq : Int32 = 0) : Int32
      Proc(Handle, Int32, Int32).new(sym("shainet_kv_cache_len"), Pointer(Void).null).call(cache, seq)
    end

    def kv_cache_capacity(cache : Handle) : Int32
      Proc(Handle, Int32).new(sym("shainet_kv_cache_capacity"), Pointer(Void).null).call(cache)
    end

    def kv_cache_reserve(cache : Handle, capacity : Int32)
      fn = Proc(Handle, Int32, Int32).new(sym("shainet_kv_cache_reserve"), Pointer(Void).null)
      status = fn.call(cache, capacity)
      if status == 3
        GC.collect
        status = fn.call(cache, capacity)
      end
      check(status)
    end

    # RoPE.apply (src/shainet/transformer/rope.cr:7-33) on host rows: [seq_len, head_dim] in and out.
    def rope_apply(x : Pointer(Float32), out_ptr : Pointer(Float32), seq_len : Int32, head_dim : Int32,
                   start_pos : Int32, theta : Float64)
      fn = Proc(Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Float64, Int32, Int32).new(sym("shainet_rope_apply"), Pointer(Void).null)
      check fn.call(x, out_ptr, seq_len, head_dim, start_pos, theta, MEM_HOST)
    end

    # y[rows, n] = x[rows, k] W[k, n] (+ res) on device pointers: what LlamaBlock#gpu_matmul dispatches
    # (llama_block.cr:726-768); stream null = the default stream.
    def matmul_f32(x : Pointer(Float32), x_stride : Int64, w : Pointer(Float32), res : Pointer(Float32),
                   y : Pointer(Float32), rows : Int32, k : Int32, n : Int32, stream : Pointer(Void) = Pointer(Void).null)
      fn = Proc(Pointer(Float32), Int64, Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32, Int32, Pointer(Void), Int32).new(sym("shainet_hip_matmul_f32"), Pointer(Void).null)
      check fn.call(x, x_stride, w, res, y, rows, k, n, stream)
    end

    # Decode calls on device pointers that allocate nothing (graph capture, tight serving loops):
    # shainet_attn_forward_noalloc.  One sequence (cache slot 0), new_tokens rows.
    def attn_forward_noalloc(ctx : Handle, cache : Handle, new_tokens : Int32,
                             q : Pointer(Float32), k : Pointer(Float32), v : Pointer(Float32), out_ptr : Pointer(Float32))
      fn = Proc(Handle, Handle, Pointer(Int32), Pointer(Int32), Int32, Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32).new(sym("shainet_attn_forward_noalloc"), Pointer(Void).null)
      nt = new_tokens
      check fn.call(ctx, cache, Pointer(Int32).null, pointerof(nt), 1, q, k, v, out_ptr)
    end

    # Decode steps with the cached lengths on the device (launches that never change: a step can be
    # recorded into a HIP graph and replayed): shainet_kv_cache_lengths_to_device before the first
    # step, shainet_attn_decode_step per token, shainet_kv_cache_lengths_from_device after the last.
    def kv_cache_lengths_to_device(cache : Handle)
      check Proc(Handle, Int32).new(sym("shainet_kv_cache_lengths_to_device"), Pointer(Void).null).call(cache)
    end

    def kv_cache_lengths_from_device(cache : Handle)
      check Proc(Handle, Int32).new(sym("shainet_kv_cache_lengths_from_device"), Pointer(Void).null).call(cache)
    end

    def attn_decode_step(ctx : Handle, cache : Handle, n_seqs : Int32,
                         q : Pointer(Float32), k : Pointer(Float32), v : Pointer(Float32), out_ptr : Pointer(Float32))
      fn = Proc(Handle, Handle, Int32, Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32).new(sym("shainet_attn_decode_step"), Pointer(Void).null)
      check fn.call(ctx, cache, n_seqs, q, k, v, out_ptr)
    end

    def attn_sync(ctx : Handle)
      check Proc(Handle, Int32).new(sym("shainet_attn_sync"), Pointer(Void).null).call(ctx)
    end

    # Host-pointer mode: q, k, v and out are SimpleMatrix buffers; returns with out filled.
    def attn_forward(ctx : Handle, cache : Handle, new_tokens : Int32,
                     q : Pointer(Float32), k : Pointer(Float32), v : Pointer(Float32), out_ptr : Pointer(Float32))
      fn = Proc(Handle, Handle, Pointer(Int32), Pointer(Int32), Int32, Pointer(Float32), Pointer(Float32), Pointer(Float32), Pointer(Float32), Int32, Int32).new(sym("shainet_attn_forward"), Pointer(Void).null)
      nt = new_tokens
      check fn.call(ctx, cache, Pointer(Int32).null, pointerof(nt), 1, q, k, v, out_ptr, MEM_HOST)
    end
  end
end
