// SafeTensors reader on the host: SHAInet::SafeTensors::File and ShardedFile
// (src/shainet/safetensors.cr) over memory-mapped files, and HFLoader.open_safetensors
// (src/shainet/hf_loader.cr:9-26).  Nothing here touches the GPU.
#include "safetensors.hpp"

#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <new>

#include "../../include/shainet_hip_attn.h"
#include "mini_json.hpp"

void shainet_hip_set_error(int code, const char *msg);  // capi.hip

namespace shainet {

int dtype_size(const std::string &d) {
  if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
  if (d == "F32" || d == "I32" || d == "U32") return 4;
  if (d == "F64" || d == "I64" || d == "U64") return 8;
  if (d == "I8" || d == "U8" || d == "BOOL") return 1;
  return 0;
}

namespace {

int fail(int code, const std::string &msg) {
  shainet_hip_set_error(code, msg.c_str());
  return code;
}

bool file_exists(const std::string &p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}
bool dir_exists(const std::string &p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

int map_file(const std::string &path, StMapping &m) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) return fail(SHAINET_HIP_ERR_ARGUMENT, "cannot open " + path);
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 8) {
    close(fd);
    return fail(SHAINET_HIP_ERR_ARGUMENT, path + " is not a SafeTensors file (shorter than its header size field)");
  }
  void *p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (p == MAP_FAILED) return fail(SHAINET_HIP_ERR_RUNTIME, "mmap failed for " + path);
  m.base = p;
  m.size = (size_t)st.st_size;
  return SHAINET_HIP_OK;
}

// One file: parse its header and append its tensors.
int add_file(shainet_safetensors *st, const std::string &path) {
  StMapping m;
  int rc = map_file(path, m);
  if (rc) return rc;
  st->maps.push_back(m);
  const unsigned char *base = (const unsigned char *)m.base;
  uint64_t header_size = 0;
  for (int i = 7; i >= 0; --i) header_size = (header_size << 8) | base[i];
  if (header_size > 100000000ull)  // safetensors.cr:52
    return fail(SHAINET_HIP_ERR_ARGUMENT, "SafeTensors header too large: " + std::to_string(header_size) + " bytes");
  if (8 + header_size > m.size) return fail(SHAINET_HIP_ERR_ARGUMENT, path + ": header runs past the end of the file");
  Json header;
  std::string err;
  if (!JsonParser((const char *)base + 8, (size_t)header_size).parse(header, err) || header.kind != Json::kObject)
    return fail(SHAINET_HIP_ERR_ARGUMENT, path + ": " + (err.empty() ? "header is not a JSON object" : err));
  const size_t data_off = 8 + (size_t)header_size;
  for (const auto &kv : header.obj) {
    if (kv.first == "__metadata__") continue;
    const Json *dt = kv.second.get("dtype"), *sh = kv.second.get("shape"), *off = kv.second.get("data_offsets");
    if (!dt || dt->kind != Json::kString || !sh || sh->kind != Json::kArray || !off || off->kind != Json::kArray ||
        off->arr.size() != 2)
      return fail(SHAINET_HIP_ERR_ARGUMENT, path + ": malformed entry for tensor '" + kv.first + "'");
    StTensor t;
    t.name = kv.first;
    t.dtype = dt->str;
    for (const Json &d : sh->arr) t.shape.push_back(d.inum);
    const long long b = off->arr[0].inum, e = off->arr[1].inum;
    if (b < 0 || e < b || data_off + (size_t)e > m.size)
      return fail(SHAINET_HIP_ERR_ARGUMENT, path + ": data of tensor '" + kv.first + "' lies outside the file");
    t.data = base + data_off + b;
    t.nbytes = e - b;
    st->index[t.name] = (int)st->tensors.size();
    st->tensors.push_back(std::move(t));
  }
  return SHAINET_HIP_OK;
}

}  // namespace
}  // namespace shainet

using namespace shainet;

extern "C" {

int shainet_safetensors_close(shainet_safetensors *st) {
  if (!st) return SHAINET_HIP_OK;
  for (StMapping &m : st->maps)
    if (m.base) munmap(m.base, m.size);
  delete st;
  return SHAINET_HIP_OK;
}

int shainet_safetensors_open(const char *path, shainet_safetensors **out) {
  if (!out) return fail(SHAINET_HIP_ERR_ARGUMENT, "out is null");
  *out = nullptr;
  if (!path) return fail(SHAINET_HIP_ERR_ARGUMENT, "path is null");
  shainet_safetensors *st = new (std::nothrow) shainet_safetensors();
  if (!st) return fail(SHAINET_HIP_ERR_ALLOC, "out of host memory");
  int rc = SHAINET_HIP_OK;
  const std::string p(path);
  if (dir_exists(p)) {  // HFLoader.open_safetensors
    const std::string single = p + "/model.safetensors", index = p + "/model.safetensors.index.json";
    if (file_exists(single)) {
      rc = add_file(st, single);
    } else if (file_exists(index)) {
      StMapping m;
      rc = map_file(index, m);
      if (!rc) {
        Json j;
        std::string err;
        const bool ok = JsonParser((const char *)m.base, m.size).parse(j, err);
        munmap(m.base, m.size);
        const Json *wm = ok ? j.get("weight_map") : nullptr;
        if (!wm || wm->kind != Json::kObject) {
          rc = fail(SHAINET_HIP_ERR_ARGUMENT, index + ": no weight_map object" + (err.empty() ? "" : " (" + err + ")"));
        } else {
          // every shard once, in the order the map first names it; a tensor belongs to the shard the map says
          std::vector<std::string> shards;
          for (const auto &kv : wm->obj) {
            bool seen = false;
            for (const std::string &s : shards) seen = seen || s == kv.second.str;
            if (!seen) shards.push_back(kv.second.str);
          }
          shainet_safetensors all;
          std::vector<size_t> first_of_shard;
          for (size_t i = 0; i < shards.size() && !rc; ++i) {
            first_of_shard.push_back(all.tensors.size());
            rc = add_file(&all, p + "/" + shards[i]);
          }
          first_of_shard.push_back(all.tensors.size());
          for (const auto &kv : wm->obj) {
            if (rc) break;
            size_t si = 0;
            while (shards[si] != kv.second.str) ++si;
            int found = -1;
            for (size_t t = first_of_shard[si]; t < first_of_shard[si + 1]; ++t)
              if (all.tensors[t].name == kv.first) found = (int)t;
            if (found < 0) {
              rc = fail(SHAINET_HIP_ERR_ARGUMENT, "Tensor '" + kv.first + "' not found in shard " + kv.second.str);
            } else {
              st->index[kv.first] = (int)st->tensors.size();
              st->tensors.push_back(all.tensors[found]);
            }
          }
          st->maps = all.maps;  // the mappings now belong to st
          all.maps.clear();
        }
      }
    } else {
      rc = fail(SHAINET_HIP_ERR_ARGUMENT,
                "No model.safetensors or model.safetensors.index.json found in " + p);  // hf_loader.cr:24
    }
  } else {
    rc = add_file(st, p);
  }
  if (rc) {
    shainet_safetensors_close(st);
    return rc;
  }
  *out = st;
  return SHAINET_HIP_OK;
}

int shainet_safetensors_count(const shainet_safetensors *st) { return st ? (int)st->tensors.size() : -1; }

const char *shainet_safetensors_name(const shainet_safetensors *st, int i) {
  if (!st || i < 0 || i >= (int)st->tensors.size()) return nullptr;
  return st->tensors[i].name.c_str();
}

int shainet_safetensors_has(const shainet_safetensors *st, const char *name) {
  return st && name && st->find(name) ? 1 : 0;
}

int shainet_safetensors_info(const shainet_safetensors *st, const char *name, char dtype[8], long long shape[8],
                             int *ndim, long long *nbytes) {
  if (!st || !name) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  const StTensor *t = st->find(name);
  if (!t) return fail(SHAINET_HIP_ERR_ARGUMENT, std::string("Tensor '") + name + "' not found");
  if (dtype) {
    memset(dtype, 0, 8);
    strncpy(dtype, t->dtype.c_str(), 7);
  }
  if (ndim) *ndim = (int)t->shape.size();
  if (shape)
    for (size_t i = 0; i < t->shape.size() && i < 8; ++i) shape[i] = t->shape[i];
  if (nbytes) *nbytes = t->nbytes;
  return SHAINET_HIP_OK;
}

int shainet_safetensors_read_f32(const shainet_safetensors *st, const char *name, float *out, long long n) {
  if (!st || !name || !out) return fail(SHAINET_HIP_ERR_ARGUMENT, "null argument");
  const StTensor *t = st->find(name);
  if (!t) return fail(SHAINET_HIP_ERR_ARGUMENT, std::string("Tensor '") + name + "' not found");
  const int es = dtype_size(t->dtype);
  const bool floaty = t->dtype == "F32" || t->dtype == "F16" || t->dtype == "BF16" || t->dtype == "F64";
  if (!floaty)  // safetensors.cr:121
    return fail(SHAINET_HIP_ERR_ARGUMENT, "Unsupported dtype " + t->dtype + " for float conversion");
  const long long count = t->nbytes / es;
  if (n != count)
    return fail(SHAINET_HIP_ERR_ARGUMENT, std::string("tensor '") + name + "' holds " + std::to_string(count) +
                                              " values, the buffer " + std::to_string(n));
  const unsigned char *p = t->data;
  if (t->dtype == "F32") {
    memcpy(out, p, (size_t)count * 4);
  } else if (t->dtype == "F64") {
    for (long long i = 0; i < count; ++i) {
      double d;
      memcpy(&d, p + 8 * i, 8);
      out[i] = (float)d;
    }
  } else {
    const bool half = t->dtype == "F16";
    for (long long i = 0; i < count; ++i) {
      uint16_t b;
      memcpy(&b, p + 2 * i, 2);
      const uint32_t w = half ? f16_bits_to_f32_bits(b) : bf16_bits_to_f32_bits(b);
      memcpy(&out[i], &w, 4);
    }
  }
  return SHAINET_HIP_OK;
}

}  // extern "C"
