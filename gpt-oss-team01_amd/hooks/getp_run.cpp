// Drop-in replacement for the reference's getp-csrc/getp_run.cpp: the three hooks that
// getp-csrc/getp_eval.cpp:97-100 declares and getp() calls (getp_eval.cpp:102-145), implemented on
// the C ABI of libgptoss_mi355.so.  Like the file it replaces it is #included by run.cpp
// (run.cpp:1072), so it sees the reference's Transformer, Tokenizer, Sampler and Requests types.
//
//   warm_up   : uploads the mmap'd fp32 checkpoint into the engine's device layout (untimed)
//   inference : tokenises the requests with the reference's encode(), runs the lock-step greedy
//               decode loop, fills Requests.tok_gens (rows of max_seq_len+1 ints, -1 terminated)
//               and returns the generated-token count the harness divides by the elapsed time
//   finish    : frees the engine
//
// Failures print the library's error text and exit, which is what the reference's hooks do
// (getp-csrc/include/tensor.hpp:20-27, getp_run.cpp:28-32).
//
// Knobs (environment): GPTOSS_BATCH = sequences decoded in lock step (default 1024; the reference
// uses 896 per GPU, getp-csrc/include/config.hpp:16-19).
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "gptoss_mi355.h"

static gptoss_engine *g_gptoss_engine = nullptr;
static int g_gptoss_max_seq = 0;

static void gptoss_die(const char *what) {
  fprintf(stderr, "gptoss_mi355: %s: %s\n", what, gptoss_last_error_string());
  exit(EXIT_FAILURE);
}

void warm_up(Transformer *transformer, Tokenizer *tokenizer) {
  (void)tokenizer;
  static_assert(sizeof(Config) == sizeof(gptoss_config), "checkpoint header layout changed");
  gptoss_config cfg;
  memcpy(&cfg, &transformer->config, sizeof(cfg));
  const float *weights = transformer->data + sizeof(Config) / sizeof(float);
  const char *env = getenv("GPTOSS_BATCH");
  int max_batch = env ? atoi(env) : 1024;
  if (max_batch < 1) max_batch = 1;
  // the reference caps the context at 1024 positions (getp-csrc/src/alloc.cpp:1047)
  g_gptoss_max_seq = cfg.seq_len < 1024 ? cfg.seq_len : 1024;
  // GPTOSS_PRECISE=1: the CPU model's fp32/double arithmetic on the GPU (exact greedy ids, slow)
  const char *precise = getenv("GPTOSS_PRECISE");
  const char *lockstep = getenv("GPTOSS_NO_PREFILL");  // prompts one position per step, as the reference
  // GPTOSS_MXFP4=1: experts stored in MXFP4 (exact for GPT-OSS checkpoints, a quarter of the bytes)
  const char *mxfp4 = getenv("GPTOSS_MXFP4");
  const int flags = ((precise && atoi(precise) != 0) ? GPTOSS_ENGINE_PRECISE : 0) |
                    ((lockstep && atoi(lockstep) != 0) ? GPTOSS_ENGINE_NO_PREFILL : 0) |
                    ((mxfp4 && atoi(mxfp4) != 0) ? GPTOSS_ENGINE_MXFP4_EXPERTS : 0);
  if (gptoss_engine_create(&cfg, weights, max_batch, g_gptoss_max_seq, flags, 0, &g_gptoss_engine) != GPTOSS_OK)
    gptoss_die("engine_create");
}

void finish(Transformer *transformer, Tokenizer *tokenizer) {
  (void)transformer;
  (void)tokenizer;
  gptoss_engine_destroy(g_gptoss_engine);
  g_gptoss_engine = nullptr;
}

long long inference(Transformer *transformer, Tokenizer *tokenizer, Sampler *sampler,
                    Requests *requests) {
  (void)sampler;  // greedy arg-max, as the reference's GPU path (model.cpp:146-148)
  const int n_req = requests->num_reqs;
  int max_seq_len = requests->max_seq_len;
  if (max_seq_len > g_gptoss_max_seq + 1) {
    fprintf(stderr, "gptoss_mi355: %d steps requested, engine holds %d positions\n", max_seq_len,
            g_gptoss_max_seq);
    exit(EXIT_FAILURE);
  }
  // tokenise on the host with the reference's encoder (getp_run_submit.cpp:32-48)
  std::vector<std::vector<int>> toks(n_req);
  std::vector<int> n_prompt(n_req);
  int stride = 1;
  for (int i = 0; i < n_req; i++) {
    const char *text = get_str_req_ptr(requests, i);
    if (!text) text = "";
    std::vector<int> buf(strlen(text) + 3);
    int count = 0;
    encode(tokenizer, text, -1, -1, buf.data(), &count, transformer->config.initial_context_length);
    if (count < 1) {
      fprintf(stderr, "something is wrong, expected at least 1 prompt token\n");
      exit(EXIT_FAILURE);
    }
    buf.resize(count);
    toks[i] = buf;
    n_prompt[i] = count;
    if (count > stride) stride = count;
  }
  std::vector<int> prompts((size_t)n_req * stride, 0);
  for (int i = 0; i < n_req; i++) memcpy(&prompts[(size_t)i * stride], toks[i].data(), sizeof(int) * toks[i].size());
  long long generated = 0;
  if (gptoss_engine_generate(g_gptoss_engine, prompts.data(), n_prompt.data(), stride, n_req, max_seq_len,
                             requests->tok_gens, &generated) != GPTOSS_OK)
    gptoss_die("engine_generate");
  return generated;
}
