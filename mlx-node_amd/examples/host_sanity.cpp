// Host-only entry points under AddressSanitizer/UBSan (no GPU needed): hyper-parameter casts, LR schedules,
// tensor layout, checkpoint header parsing with mutated inputs, null-argument refusals.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>
#include "mxopt_engine.h"

static void write_file(const char* path, const std::vector<unsigned char>& bytes) {
  FILE* f = fopen(path, "wb");
  fwrite(bytes.data(), 1, bytes.size(), f);
  fclose(f);
}

int main() {
  mxopt_adam_hp a; mxopt_adam_hp_from_f64(1e-3, 0.9, 0.999, 1e-8, 0.01, 1, &a);
  mxopt_sgd_hp s; if (mxopt_sgd_hp_from_f64(0.1, 0.0, 0.0, 0.0, 1, &s) == 0) return 1;
  mxopt_rmsprop_hp r; mxopt_rmsprop_hp_from_f64(1e-3, 0.99, 1e-8, 0.0, &r);
  float b1, b2; mxopt_bias_correction(0.9, 0.999, 7, &b1, &b2);
  volatile double sink = mxopt_lr_linear_decay(1, 0.1, 50, 100) + mxopt_lr_exponential_decay(1, 0.9, 25, 10) +
                         mxopt_lr_cosine_annealing(1, 0.1, 50, 100) + mxopt_lr_step_decay(1, 0.5, 31, 10);
  (void)sink;
  for (uintptr_t k = 0; k < 64; ++k) {
    mxopt_tensor t; memset(&t, 0, sizeof t);
    t.p = (void*)(0x7f0000000000ull + 2 * k); t.p_out = (void*)t.p; t.g = (void*)(0x7e0000000000ull + 2 * (k % 5));
    t.m = (float*)(0x7d0000000000ull + 4 * k); t.n = 100000 + k; t.p_dtype = t.p_out_dtype = t.g_dtype = MXOPT_BF16;
    uint32_t head; int vec; uint64_t nc;
    if (mxopt_tensor_layout(&t, &head, &vec, &nc)) return 2;
  }
  if (mxopt_engine_micro_batch(nullptr, 0, nullptr, nullptr, nullptr) == 0) return 3;
  if (mxopt_optimizer_update_single(nullptr, "x", nullptr, nullptr, nullptr) == 0) return 4;
  mxopt_engine_config cfg; mxopt_engine_config_default(MXOPT_ENGINE_SFT, &cfg);

  // checkpoint headers: a valid one, then 20000 mutations
  const std::string header = "{\"a.m\":{\"dtype\":\"F32\",\"shape\":[8],\"data_offsets\":[0,32]},\"a.v\":{\"dtype\":\"F32\",\"shape\":[8],"
                             "\"data_offsets\":[32,64]},\"__metadata__\":{\"format\":\"mxopt-optimizer-state\",\"optimizer\":\"adamw\",\"step\":\"12\"}}";
  std::vector<unsigned char> good(8 + header.size() + 64, 0);
  const uint64_t hlen = header.size();
  memcpy(good.data(), &hlen, 8);
  memcpy(good.data() + 8, header.data(), header.size());
  const char* path = "/tmp/mxopt_asan_ckpt.bin";
  write_file(path, good);
  char kind[8]; int64_t step; uint64_t nt, ne;
  if (mxopt_checkpoint_inspect(path, kind, sizeof kind, &step, &nt, &ne) != 0 || step != 12 || nt != 2 || ne != 16) return 5;
  unsigned seed = 12345;
  int accepted = 0;
  for (int it = 0; it < 20000; ++it) {
    std::vector<unsigned char> bad = good;
    const int flips = 1 + rand_r(&seed) % 4;
    for (int f = 0; f < flips; ++f) bad[rand_r(&seed) % bad.size()] = (unsigned char)rand_r(&seed);
    if (rand_r(&seed) % 8 == 0) bad.resize(rand_r(&seed) % bad.size());
    write_file(path, bad);
    if (mxopt_checkpoint_inspect(path, kind, sizeof kind, &step, &nt, &ne) == 0) {
      ++accepted;
      if (ne * 4 > bad.size()) return 6;
    }
  }
  printf("host sanity ok (%d of 20000 mutated headers still valid)\n", accepted);
  return 0;
}
