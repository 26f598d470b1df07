/* The C ABI called from plain C, as a host written in a compiled language would call it
 * (the reference binds its kernel library with dlopen + dlsym, src/shainet/cuda.cr:281-309,
 * 841-852).  No oracle here: the answers are closed forms.
 *   - first row of a sequence: one visible key, so every head's output is its kv head's V row;
 *   - second row: a softmax over two keys, recomputed here in double from the same rotation
 *     (half-split RoPE, angle = pos * theta^(-2i/hd), llama_block.cr:266-286 and 332-344);
 *   - the lengths, the capacity error (nothing appended) and the size check of the biases.
 * Exit status 0 when everything holds; a message on stderr otherwise. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../include/shainet_hip_attn.h"

#define H 8
#define KV 2
#define HD 64
#define G (H / KV)

static int failures = 0;
#define CHECK(cond, ...)                  \
  do {                                    \
    if (!(cond)) {                        \
      fprintf(stderr, "cabi_smoke: ");    \
      fprintf(stderr, __VA_ARGS__);       \
      fprintf(stderr, "\n");              \
      ++failures;                         \
    }                                     \
  } while (0)

static unsigned long long rng_state = 88172645463325252ULL;
static float rnd(void) { /* xorshift, uniform in [-1, 1) */
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 7;
  rng_state ^= rng_state << 17;
  return (float)((double)(rng_state >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

static void rotate(const float *x, int pos, double theta, double *out) {
  for (int i = 0; i < HD / 2; ++i) {
    const float freq = (float)(1.0 / pow(theta, 2.0 * i / HD));
    const float angle = (float)pos * freq;
    const double c = cosf(angle), s = sinf(angle);
    out[i] = x[i] * c - x[i + HD / 2] * s;
    out[i + HD / 2] = x[i + HD / 2] * c + x[i] * s;
  }
}

int main(void) {
  if (!shainet_hip_available()) {
    fprintf(stderr, "cabi_smoke: no gfx950 device\n");
    return 2;
  }
  const double theta = 10000.0;
  shainet_attn_ctx *ctx = NULL;
  shainet_kv_cache *cache = NULL;
  shainet_attn_ctx *refused = NULL;
  CHECK(shainet_attn_create(&refused, 7, 2, HD, theta, NULL, NULL, 0, NULL, 0, 1e-6, 64) == SHAINET_HIP_ERR_ARGUMENT &&
            refused == NULL,
        "7 heads over 2 kv heads must be refused");
  CHECK(shainet_attn_create(&ctx, H, KV, HD, theta, NULL, NULL, 0, NULL, 0, 1e-6, 64) == SHAINET_HIP_OK, "create: %s",
        shainet_hip_last_error());
  CHECK(shainet_kv_cache_create(&cache, ctx, 1, 3) == SHAINET_HIP_OK, "cache: %s", shainet_hip_last_error());
  float bias[H * HD];
  memset(bias, 0, sizeof bias);
  CHECK(shainet_attn_set_bias(ctx, bias, H * HD - 1, NULL, 0, NULL, 0) == SHAINET_HIP_ERR_ARGUMENT,
        "a bias of the wrong size must be refused");

  static float q[2][H * HD], k[2][KV * HD], v[2][KV * HD], out[H * HD];
  for (int t = 0; t < 2; ++t) {
    for (int i = 0; i < H * HD; ++i) q[t][i] = rnd();
    for (int i = 0; i < KV * HD; ++i) k[t][i] = rnd(), v[t][i] = rnd();
  }
  const int one = 1;
  /* row 0: one visible key */
  CHECK(shainet_attn_forward(ctx, cache, NULL, &one, 1, q[0], k[0], v[0], out, SHAINET_HIP_MEM_HOST) == SHAINET_HIP_OK,
        "forward: %s", shainet_hip_last_error());
  CHECK(shainet_kv_cache_len(cache, 0) == 1, "length after one row is %d", shainet_kv_cache_len(cache, 0));
  for (int h = 0; h < H; ++h)
    for (int d = 0; d < HD; ++d)
      CHECK(fabsf(out[h * HD + d] - v[0][(h / G) * HD + d]) <= 1e-6f, "row 0, head %d, d %d: %g != %g", h, d,
            out[h * HD + d], v[0][(h / G) * HD + d]);
  /* row 1: two visible keys */
  CHECK(shainet_attn_forward(ctx, cache, NULL, &one, 1, q[1], k[1], v[1], out, SHAINET_HIP_MEM_HOST) == SHAINET_HIP_OK,
        "forward: %s", shainet_hip_last_error());
  CHECK(shainet_kv_cache_len(cache, 0) == 2, "length after two rows is %d", shainet_kv_cache_len(cache, 0));
  for (int h = 0; h < H; ++h) {
    double qr[HD], k0[HD], k1[HD], s0 = 0, s1 = 0;
    rotate(q[1] + h * HD, 1, theta, qr);
    rotate(k[0] + (h / G) * HD, 0, theta, k0);
    rotate(k[1] + (h / G) * HD, 1, theta, k1);
    for (int d = 0; d < HD; ++d) s0 += qr[d] * k0[d], s1 += qr[d] * k1[d];
    s0 /= sqrt((double)HD);
    s1 /= sqrt((double)HD);
    const double mx = s0 > s1 ? s0 : s1, e0 = exp(s0 - mx), e1 = exp(s1 - mx);
    for (int d = 0; d < HD; ++d) {
      const double want = (e0 * v[0][(h / G) * HD + d] + e1 * v[1][(h / G) * HD + d]) / (e0 + e1);
      CHECK(fabs(out[h * HD + d] - want) <= 1e-4 + 1e-3 * fabs(want), "row 1, head %d, d %d: %g != %g", h, d,
            out[h * HD + d], want);
    }
  }
  /* capacity 3: two more rows do not fit, and nothing is appended */
  const int two = 2;
  static float q2[2 * H * HD], k2[2 * KV * HD], out2[2 * H * HD];
  memset(q2, 0, sizeof q2);
  memset(k2, 0, sizeof k2);
  CHECK(shainet_attn_forward(ctx, cache, NULL, &two, 1, q2, k2, k2, out2, SHAINET_HIP_MEM_HOST) == SHAINET_HIP_ERR_CAPACITY,
        "rows beyond the capacity must be refused");
  CHECK(strlen(shainet_hip_last_error()) > 0, "a refusal leaves a message");
  CHECK(shainet_kv_cache_len(cache, 0) == 2, "a refused call appended rows");
  CHECK(shainet_kv_cache_clear(cache, -1) == SHAINET_HIP_OK && shainet_kv_cache_len(cache, 0) == 0, "clear");
  CHECK(shainet_kv_cache_destroy(cache) == SHAINET_HIP_OK, "cache destroy");
  CHECK(shainet_attn_destroy(ctx) == SHAINET_HIP_OK, "destroy");
  if (failures) return 1;
  printf("cabi_smoke ok\n");
  return 0;
}
