// HFLoader.load_llama (src/shainet/hf_loader.cr:184-412) for the device: reads
// config.json, builds the model, and moves every tensor from the memory-mapped
// SafeTensors file to the GPU in its stored type (F32, F16, BF16 or F64); a
// kernel there converts it to fp32 and writes it transposed, [out, in] ->
// [in, out] (hf_loader.cr:326-337), straight into the place the decode kernels
// read: q/k/v side by side in one matrix, gate|up in another.  No fp32 copy of a
// weight matrix is ever made on the host.
#include <hip/hip_runtime.h>
#include <math.h>
#include <string.h>
#include <sys/stat.h>

#include <string>
#include <vector>

#include "../../include/shainet_hip_attn.h"
#include "llama_internal.hpp"
#include "mini_json.hpp"
#include "safetensors.hpp"

using namespace shainet;

namespace {

int fail(int code, const std::string &msg) { return llama_fail(code, msg); }

enum { kF32 = 0, kF16 = 1, kBF16 = 2, kF64 = 3 };

__device__ __forceinline__ float load_as_f32(const void *src, long long i, int dtype) {
  switch (dtype) {
    case kF32: return ((const float *)src)[i];
    case kF16: return __uint_as_float(f16_bits_to_f32_bits(((const unsigned short *)src)[i]));
    case kBF16: return __uint_as_float(bf16_bits_to_f32_bits(((const unsigned short *)src)[i]));
    default: return (float)((const double *)src)[i];
  }
}

// dst[i] = src[i], n elements
__global__ __launch_bounds__(256) void convert_kernel(const void *__restrict__ src, float *__restrict__ dst, long long n,
                                                      int dtype) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = load_as_f32(src, i, dtype);
}

// src [rows, cols] row-major -> dst[c * ld + r] for every (r, c): the transpose, written into a
// matrix whose rows are ld floats long (dst already points at the first column to fill).
// 32 x 32 tiles through LDS so that both the reads and the writes are coalesced.
__global__ __launch_bounds__(256) void convert_transpose_kernel(const void *__restrict__ src, float *__restrict__ dst,
                                                                int rows, int cols, long long ld, int dtype) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
  for (int j = 0; j < 32; j += 8) {
    const int r = r0 + ty + j, c = c0 + tx;
    if (r < rows && c < cols) tile[ty + j][tx] = load_as_f32(src, (long long)r * cols + c, dtype);
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 32; j += 8) {
    const int c = c0 + ty + j, r = r0 + tx;
    if (r < rows && c < cols) dst[(long long)c * ld + r] = tile[tx][ty + j];
  }
}

// dst[c * ld + r] = src[r * cols + c] for fp32 already on the device (tied lm_head = embedding^T)
int dtype_code(const std::string &d) {
  if (d == "F32") return kF32;
  if (d == "F16") return kF16;
  if (d == "BF16") return kBF16;
  if (d == "F64") return kF64;
  return -1;
}

struct Stager {
  void *dev = nullptr;
  size_t cap = 0;
  ~Stager() {
    if (dev) (void)hipFree(dev);
  }
  int put(const StTensor &t) {
    if ((size_t)t.nbytes > cap) {
      if (dev) (void)hipFree(dev);
      dev = nullptr;
      cap = 0;
      if (hipMalloc(&dev, (size_t)t.nbytes) != hipSuccess) return fail(SHAINET_HIP_ERR_ALLOC, "hipMalloc failed");
      cap = (size_t)t.nbytes;
    }
    // pageable (memory-mapped) source: returns when the bytes have left the mapping
    if (hipMemcpy(dev, t.data, (size_t)t.nbytes, hipMemcpyHostToDevice) != hipSuccess)
      return fail(SHAINET_HIP_ERR_RUNTIME, "hipMemcpy of tensor '" + t.name + "' failed");
    return SHAINET_HIP_OK;
  }
};

const StTensor *need(const shainet_safetensors *st, const std::string &name, int &rc) {
  const StTensor *t = st->find(name);
  if (!t) rc = fail(SHAINET_HIP_ERR_ARGUMENT, "Tensor '" + name + "' not found");
  return t;
}

// A [rows, cols] tensor (1-D: one row), checked against the shape the model expects.
int check_matrix(const StTensor &t, long long rows, long long cols, int &dtype) {
  dtype = dtype_code(t.dtype);
  if (dtype < 0) return fail(SHAINET_HIP_ERR_ARGUMENT, "Unsupported dtype " + t.dtype + " for float conversion");
  if (t.shape.size() > 2)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "Cannot read tensor '" + t.name + "' with " + std::to_string(t.shape.size()) +
                                              "D shape as matrix");
  const long long r = t.shape.size() == 2 ? t.shape[0] : 1, c = t.shape.empty() ? 1 : t.shape.back();
  if (r != rows || c != cols || t.nbytes != rows * cols * dtype_size(t.dtype))
    return fail(SHAINET_HIP_ERR_ARGUMENT, "tensor '" + t.name + "' is [" + std::to_string(r) + ", " + std::to_string(c) +
                                              "], the model needs [" + std::to_string(rows) + ", " +
                                              std::to_string(cols) + "]");
  return SHAINET_HIP_OK;
}

// HF [out, in] tensor -> columns [col0, col0 + out) of the device matrix dst [in, ld]
int load_transposed(const shainet_safetensors *st, Stager &stage, const std::string &name, int out_dim, int in_dim,
                    float *dst, long long ld, long long col0) {
  int rc = SHAINET_HIP_OK, dtype;
  const StTensor *t = need(st, name, rc);
  if (!t) return rc;
  if ((rc = check_matrix(*t, out_dim, in_dim, dtype)) || (rc = stage.put(*t))) return rc;
  dim3 grid((unsigned)((in_dim + 31) / 32), (unsigned)((out_dim + 31) / 32));
  hipLaunchKernelGGL(convert_transpose_kernel, grid, dim3(256), 0, nullptr, stage.dev, dst + col0, out_dim, in_dim, ld,
                     dtype);
  if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess)  // the staging buffer is reused next
    return fail(SHAINET_HIP_ERR_RUNTIME, "converting tensor '" + name + "' failed");
  return SHAINET_HIP_OK;
}

int load_plain(const shainet_safetensors *st, Stager &stage, const std::string &name, long long rows, long long cols,
               float *dst) {
  int rc = SHAINET_HIP_OK, dtype;
  const StTensor *t = need(st, name, rc);
  if (!t) return rc;
  if ((rc = check_matrix(*t, rows, cols, dtype)) || (rc = stage.put(*t))) return rc;
  const long long n = rows * cols;
  hipLaunchKernelGGL(convert_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, nullptr, stage.dev, dst, n, dtype);
  if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess)
    return fail(SHAINET_HIP_ERR_RUNTIME, "converting tensor '" + name + "' failed");
  return SHAINET_HIP_OK;
}

int read_host_vector(const shainet_safetensors *st, const std::string &name, std::vector<float> &out) {
  const StTensor *t = st->find(name);
  if (!t) return fail(SHAINET_HIP_ERR_ARGUMENT, "Tensor '" + name + "' not found");
  const int es = dtype_size(t->dtype);
  out.resize(es ? (size_t)(t->nbytes / es) : 0);
  return shainet_safetensors_read_f32(st, name.c_str(), out.data(), (long long)out.size());
}

bool as_int(const Json *j, int &v) {
  if (!j || j->kind != Json::kNumber) return false;
  v = (int)j->inum;
  return true;
}
bool as_double(const Json *j, double &v) {
  if (!j || j->kind != Json::kNumber) return false;
  v = j->num;
  return true;
}

int read_text(const std::string &path, std::string &out) {
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) return fail(SHAINET_HIP_ERR_ARGUMENT, "config.json not found in " + path.substr(0, path.rfind('/')));
  char buf[4096];
  size_t n;
  out.clear();
  while ((n = fread(buf, 1, sizeof buf, f)) > 0) out.append(buf, n);
  fclose(f);
  return SHAINET_HIP_OK;
}

}  // namespace

extern "C" {

int shainet_hf_read_llama_config(const char *model_dir, shainet_hf_llama_config *cfg) {
  if (!model_dir || !cfg) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  memset(cfg, 0, sizeof *cfg);
  std::string text, err;
  int rc = read_text(std::string(model_dir) + "/config.json", text);
  if (rc) return rc;
  Json j;
  if (!JsonParser(text.data(), text.size()).parse(j, err) || j.kind != Json::kObject)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "config.json: " + (err.empty() ? std::string("not a JSON object") : err));
  const Json *mt = j.get("model_type");
  if (!mt || mt->kind != Json::kString) return fail(SHAINET_HIP_ERR_ARGUMENT, "No model_type in config.json");
  strncpy(cfg->model_type, mt->str.c_str(), sizeof cfg->model_type - 1);
  // load_llama_config (hf_loader.cr:215-233)
  if (!as_int(j.get("vocab_size"), cfg->vocab_size) || !as_int(j.get("hidden_size"), cfg->hidden_size) ||
      !as_int(j.get("num_attention_heads"), cfg->num_attention_heads) ||
      !as_int(j.get("num_hidden_layers"), cfg->num_hidden_layers) ||
      !as_int(j.get("intermediate_size"), cfg->intermediate_size) || !as_double(j.get("rms_norm_eps"), cfg->rms_norm_eps))
    return fail(SHAINET_HIP_ERR_ARGUMENT,
                "config.json lacks one of vocab_size, hidden_size, num_attention_heads, num_hidden_layers, "
                "intermediate_size, rms_norm_eps");
  cfg->rope_theta = 10000.0;
  if (!as_double(j.get("rope_theta"), cfg->rope_theta)) {
    const Json *rp = j.get("rope_parameters");
    if (rp) as_double(rp->get("rope_theta"), cfg->rope_theta);
  }
  if (!as_int(j.get("num_key_value_heads"), cfg->num_key_value_heads)) cfg->num_key_value_heads = cfg->num_attention_heads;
  const Json *tie = j.get("tie_word_embeddings");
  cfg->tie_word_embeddings = tie && tie->kind == Json::kBool && tie->b ? 1 : 0;
  as_int(j.get("head_dim"), cfg->head_dim);  // stays 0 when absent or null
  if (!as_int(j.get("num_experts"), cfg->num_experts)) as_int(j.get("num_local_experts"), cfg->num_experts);
  // compute_rope_freqs (235-242): only rope_scaling of type "llama3" changes the frequencies
  const Json *rs = j.get("rope_scaling");
  if (rs && rs->kind == Json::kObject) {
    const Json *ty = rs->get("rope_type");
    if (!ty || ty->kind != Json::kString) ty = rs->get("type");
    if (ty && ty->kind == Json::kString && ty->str == "llama3") {
      int old_ctx = 0;
      if (!as_double(rs->get("factor"), cfg->rope_factor) || !as_double(rs->get("low_freq_factor"), cfg->rope_low_freq_factor) ||
          !as_double(rs->get("high_freq_factor"), cfg->rope_high_freq_factor) ||
          !as_int(rs->get("original_max_position_embeddings"), old_ctx))
        return fail(SHAINET_HIP_ERR_ARGUMENT, "config.json: incomplete llama3 rope_scaling");
      cfg->rope_original_max_position_embeddings = old_ctx;
      cfg->rope_llama3 = 1;
    }
  }
  return SHAINET_HIP_OK;
}

int shainet_hf_rope_freqs(const shainet_hf_llama_config *cfg, float *out, int n) {
  if (!cfg || !out) return -fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  if (cfg->num_attention_heads < 1) return -fail(SHAINET_HIP_ERR_ARGUMENT, "num_attention_heads must be positive");
  const int head_dim = cfg->head_dim ? cfg->head_dim : cfg->hidden_size / cfg->num_attention_heads;
  if (!cfg->rope_llama3) return 0;  // nil: the block uses theta^(-2i/d)
  if (n != head_dim / 2) return -fail(SHAINET_HIP_ERR_ARGUMENT, "out must hold head_dim / 2 values");
  // hf_loader.cr:244-265, all in fp64, rounded once
  const double theta = cfg->rope_theta, factor = cfg->rope_factor;
  const double old_ctx = (double)cfg->rope_original_max_position_embeddings;
  const double low_freq_wavelen = old_ctx / cfg->rope_low_freq_factor;
  const double high_freq_wavelen = old_ctx / cfg->rope_high_freq_factor;
  for (int i = 0; i < head_dim / 2; ++i) {
    const double inv = 1.0 / pow(theta, 2.0 * i / head_dim);
    const double wavelen = 2.0 * M_PI / inv;
    double new_inv;
    if (wavelen < high_freq_wavelen) {
      new_inv = inv;
    } else if (wavelen > low_freq_wavelen) {
      new_inv = inv / factor;
    } else {
      const double smooth = (old_ctx / wavelen - cfg->rope_low_freq_factor) / (cfg->rope_high_freq_factor - cfg->rope_low_freq_factor);
      new_inv = (1.0 - smooth) * inv / factor + smooth * inv;
    }
    out[i] = (float)new_inv;
  }
  return head_dim / 2;
}

int shainet_hf_load_llama(const char *model_dir, shainet_llama_model **out) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  shainet_hf_llama_config cfg;
  int rc = shainet_hf_read_llama_config(model_dir, &cfg);
  if (rc) return rc;
  const std::string mt = cfg.model_type;
  if (mt == "qwen3_moe" || cfg.num_experts > 0)
    return fail(SHAINET_HIP_ERR_ARGUMENT, "mixture-of-experts models (" + mt + ") are not covered by this loader");
  if (mt != "llama" && mt != "mistral" && mt != "qwen2" && mt != "qwen3")  // hf_loader.cr:38-45
    return fail(SHAINET_HIP_ERR_ARGUMENT, "Unsupported model_type: '" + mt + "'. Supported: llama, mistral, qwen2, qwen3");
  if (!shainet_hip_available()) return fail(SHAINET_HIP_ERR_RUNTIME, "no gfx950 device available");
  shainet_safetensors *st = nullptr;
  if ((rc = shainet_safetensors_open(model_dir, &st))) return rc;
  shainet_llama_model *m = nullptr;
  rc = shainet_llama_model_create(&m, cfg.vocab_size, cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads,
                                  cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size, cfg.rms_norm_eps,
                                  cfg.rope_theta);
  const int d = cfg.hidden_size, ff = cfg.intermediate_size, V = cfg.vocab_size;
  const int head_dim = cfg.head_dim ? cfg.head_dim : (cfg.num_attention_heads ? d / cfg.num_attention_heads : 0);
  std::vector<float> freqs(head_dim / 2 > 0 ? head_dim / 2 : 1);
  int n_freqs = 0;
  if (!rc) {
    n_freqs = shainet_hf_rope_freqs(&cfg, freqs.data(), head_dim / 2);
    if (n_freqs < 0) rc = -n_freqs;
  }
  Stager stage;
  LlamaModelBuffers mb;
  if (!rc) rc = shainet_llama_model_buffers(m, &mb);
  if (!rc) rc = load_plain(st, stage, "model.embed_tokens.weight", V, d, mb.embedding);  // [vocab, d]
  for (int li = 0; li < cfg.num_hidden_layers && !rc; ++li) {
    shainet_llama_block *b = shainet_llama_model_block(m, li);
    shainet_llama_attn *a = shainet_llama_block_attn(b);
    const std::string p = "model.layers." + std::to_string(li);
    rc = shainet_llama_attn_set_rope(a, cfg.rope_theta, n_freqs > 0 ? freqs.data() : nullptr);
    LlamaBlockBuffers bb;
    if (!rc) rc = shainet_llama_block_buffers(b, &bb);
    if (rc) break;
    const long long wide = bb.q_dim + 2LL * bb.kv_dim;
    // attention weights: HF is [out, in], the products are x * W, so [in, out] (hf_loader.cr:325-329)
    if ((rc = load_transposed(st, stage, p + ".self_attn.q_proj.weight", bb.q_dim, d, bb.w_qkv, wide, 0))) break;
    if ((rc = load_transposed(st, stage, p + ".self_attn.k_proj.weight", bb.kv_dim, d, bb.w_qkv, wide, bb.q_dim))) break;
    if ((rc = load_transposed(st, stage, p + ".self_attn.v_proj.weight", bb.kv_dim, d, bb.w_qkv, wide,
                              bb.q_dim + bb.kv_dim)))
      break;
    if ((rc = load_transposed(st, stage, p + ".self_attn.o_proj.weight", d, bb.q_dim, bb.w_o, d, 0))) break;
    // dense SwiGLU (333-336)
    if ((rc = load_transposed(st, stage, p + ".mlp.gate_proj.weight", ff, d, bb.gate_up, 2LL * ff, 0))) break;
    if ((rc = load_transposed(st, stage, p + ".mlp.up_proj.weight", ff, d, bb.gate_up, 2LL * ff, ff))) break;
    if ((rc = load_transposed(st, stage, p + ".mlp.down_proj.weight", d, ff, bb.down, d, 0))) break;
    // RMSNorm (349-350)
    if ((rc = load_plain(st, stage, p + ".input_layernorm.weight", 1, d, bb.norm1))) break;
    if ((rc = load_plain(st, stage, p + ".post_attention_layernorm.weight", 1, d, bb.norm2))) break;
    // optional Q/K/V biases, a complete set or none (352-363)
    const bool hq = st->find(p + ".self_attn.q_proj.bias"), hk = st->find(p + ".self_attn.k_proj.bias"),
               hv = st->find(p + ".self_attn.v_proj.bias");
    if (hq || hk || hv) {
      if (!(hq && hk && hv)) {
        rc = fail(SHAINET_HIP_ERR_ARGUMENT, "Incomplete Q/K/V projection biases for " + p);
        break;
      }
      std::vector<float> bq, bk, bv;
      if ((rc = read_host_vector(st, p + ".self_attn.q_proj.bias", bq)) ||
          (rc = read_host_vector(st, p + ".self_attn.k_proj.bias", bk)) ||
          (rc = read_host_vector(st, p + ".self_attn.v_proj.bias", bv)))
        break;
      if ((rc = shainet_llama_attn_set_bias(a, bq.data(), (int)bq.size(), bk.data(), (int)bk.size(), bv.data(),
                                            (int)bv.size())))
        break;
    }
    // optional Qwen3 QK-norm weights, a complete pair or none (365-375)
    const bool hqn = st->find(p + ".self_attn.q_norm.weight"), hkn = st->find(p + ".self_attn.k_norm.weight");
    if (hqn || hkn) {
      if (!(hqn && hkn)) {
        rc = fail(SHAINET_HIP_ERR_ARGUMENT, "Incomplete QK-norm weights for " + p);
        break;
      }
      std::vector<float> qn, kn;
      if ((rc = read_host_vector(st, p + ".self_attn.q_norm.weight", qn)) ||
          (rc = read_host_vector(st, p + ".self_attn.k_norm.weight", kn)))
        break;
      if ((rc = shainet_llama_attn_set_qk_norm(a, qn.data(), (int)qn.size(), kn.data(), (int)kn.size()))) break;
    }
  }
  // final RMSNorm and the output head (393-404)
  if (!rc) rc = load_plain(st, stage, "model.norm.weight", 1, d, mb.final_norm);
  if (!rc) {
    if (cfg.tie_word_embeddings) {  // embed.transpose: [d, vocab] from the rows already on the device
      dim3 grid((unsigned)((d + 31) / 32), (unsigned)((V + 31) / 32));
      hipLaunchKernelGGL(convert_transpose_kernel, grid, dim3(256), 0, nullptr, (const void *)mb.embedding, mb.lm_head, V,
                         d, (long long)V, (int)kF32);
      if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess)
        rc = fail(SHAINET_HIP_ERR_RUNTIME, "transposing the tied embedding failed");
    } else {
      rc = load_transposed(st, stage, "lm_head.weight", V, d, mb.lm_head, V, 0);
    }
  }
  shainet_safetensors_close(st);
  if (rc) {
    shainet_llama_model_destroy(m);
    return rc;
  }
  *out = m;
  return SHAINET_HIP_OK;
}

}  // extern "C"
