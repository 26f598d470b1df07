# Test double used when SHAInet is compiled without -Denable_hip: same module and
# method names as hip.cr, nothing available, every kernel call raises.  The twin
# of src/shainet/cuda_stub.cr (26-28, 97-103) for this path.
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

    alias Handle = Pointer(Void)

    def available? : Bool
      false
    end

    def kernels_available? : Bool
      false
    end

    def fully_available? : Bool
      false
    end

    {% for name in %w(malloc free memcpy device_synchronize kv_cache_append_f32 attention_kv_f32
                     attn_create attn_set_bias attn_destroy kv_cache_create kv_cache_destroy kv_cache_clear
                     kv_cache_len kv_cache_capacity kv_cache_reserve attn_forward) %}
      def {{name.id}}(*args)
        raise "HIP disabled"
      end
    {% end %}
  end
end
