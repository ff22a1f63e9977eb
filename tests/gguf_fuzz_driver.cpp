// Host-only driver of tests/test_gguf_cpu.py: seeded mutations of a small model file's header (flipped bytes,
// truncation, overwritten lengths and type ids), each parsed and fed to the model loader with the device side stubbed
// out.  Built with AddressSanitizer and UBSan: every copy of the file is a heap block of its exact size, so a read
// outside it is reported and fails the test.  usage: driver <header bytes> <trials> <file>
#include "../include/orangu_mi355x.h"
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
static uint64_t rs = 0x9E3779B97F4A7C15ull;
static uint64_t rnd() { rs ^= rs << 13; rs ^= rs >> 7; rs ^= rs << 17; return rs; }
static size_t n_uploads = 0, n_creates = 0;
extern "C" const char *ogm_last_error(ogm_ctx *) { return ""; }
extern "C" int ogm_supports(uint32_t, uint32_t) { return 1; }
extern "C" int ogm_weight_upload(ogm_ctx *, uint32_t, const void *raw, size_t row_bytes, uint32_t, uint32_t out_dim, uint64_t, uint64_t, ogm_weight **out) {
  volatile uint8_t c = 0;
  for (size_t i = 0; i < row_bytes * (size_t)out_dim; i += 97) c ^= ((const uint8_t *)raw)[i];
  if (row_bytes * (size_t)out_dim) c ^= ((const uint8_t *)raw)[row_bytes * (size_t)out_dim - 1];
  (void)c;
  n_uploads++;
  *out = (ogm_weight *)malloc(8);   // leaked on purpose: the loader documents that a failed load leaves its uploads to ogm_destroy
  return 0;
}
extern "C" int ogm_llama_create(ogm_ctx *, const ogm_llama_config *cfg, const ogm_llama_layer *layers, const float *output_norm, const ogm_weight *, ogm_llama **) {
  volatile float c = 0;
  for (uint32_t i = 0; i < cfg->n_embd; i++) c += output_norm[i];
  for (uint32_t l = 0; l < cfg->n_layer; l++) {
    for (uint32_t i = 0; i < cfg->n_embd; i++) c += layers[l].attn_norm[i] + layers[l].ffn_norm[i];
    if (layers[l].q_bias) for (uint32_t i = 0; i < cfg->n_head * cfg->head_dim; i++) c += layers[l].q_bias[i];
    if (layers[l].q_norm) for (uint32_t i = 0; i < cfg->head_dim; i++) c += layers[l].q_norm[i];
  }
  (void)c;
  n_creates++;
  return -1;
}
int main(int argc, char **argv) {
  if (argc < 4) return 2;
  FILE *f = fopen(argv[3], "rb");
  if (!f) return 2;
  std::vector<uint8_t> good;
  { uint8_t tmp[65536]; size_t n; while ((n = fread(tmp, 1, sizeof tmp, f)) > 0) good.insert(good.end(), tmp, tmp + n); }
  const size_t head = (size_t)atol(argv[1]), trials = (size_t)atol(argv[2]);
  const uint64_t big[] = {0xFFFFFFFFFFFFFFFFull, 1ull << 63, 1ull << 62, 1ull << 33, 1ull << 32, (1ull << 31) + 5, good.size(), good.size() - 1, 0, 7, 255, 65536};
  size_t parsed = 0, refused = 0, loaded_err = 0;
  for (size_t t = 0; t < trials; t++) {
    size_t len = good.size();
    const int kind = (int)(t % 6);
    if (kind == 1) len = rnd() % good.size();
    uint8_t *buf = (uint8_t *)malloc(len ? len : 1);
    memcpy(buf, good.data(), len);
    const size_t h = head < len ? head : len;
    if (h > 16) {
      if (kind == 0) for (int k = 0, n = 1 + (int)(rnd() % 5); k < n; k++) buf[rnd() % h] ^= (uint8_t)(1 + rnd() % 255);
      if (kind == 2) { const size_t p = (1 + rnd() % (h / 8 - 1)) * 8; const uint64_t v = big[rnd() % 12]; memcpy(buf + p, &v, 8); }
      if (kind == 3) { const size_t p = 4 + rnd() % (h - 12); const uint64_t v = big[rnd() % 12]; memcpy(buf + p, &v, 8); }
      if (kind == 4) { const size_t p = 4 + rnd() % (h - 8); const uint32_t v = (uint32_t)rnd(); memcpy(buf + p, &v, 4); }
      if (kind == 5) { const size_t p = 4 + rnd() % (h - 8); const uint32_t v = (uint32_t)(rnd() % 40); memcpy(buf + p, &v, 4); }
    }
    ogm_gguf *g = nullptr;
    char err[256];
    if (ogm_gguf_parse(buf, len, &g, err, sizeof err) != 0) { refused++; free(buf); continue; }
    parsed++;
    ogm_llama *model = nullptr;
    const ogm_weight *tok = nullptr;
    ogm_llama_config cfg;
    if (ogm_llama_load_gguf((ogm_ctx *)1, g, 128, &model, &tok, &cfg) != 0) loaded_err++;
    ogm_gguf_close(g);
    free(buf);
  }
  printf("parsed %zu refused %zu, loader errors %zu, uploads %zu, creates reached %zu\n", parsed, refused, loaded_err, n_uploads, n_creates);
  return 0;
}
