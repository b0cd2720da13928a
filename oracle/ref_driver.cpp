// C entry points appended to the CPU part of the reference's run.cpp when oracle/_ref is built
// (see the Makefile).  Everything called here -- build_transformer, forward, sample_argmax --
// is the reference's own code; this file only drives it with token ids instead of text, because
// the tokenizer vocabulary file cannot be produced offline.
//
// The decode loop follows the reference's getp loop (getp-csrc/submit/getp_run_submit.cpp:60-96):
// positions 0..max_seq_len-2, prompt tokens forced while pos < n_prompt-1, afterwards greedy
// arg-max stored and fed back, stop ids 199999/200002, terminator -1 at generated_len+1.

extern "C" {

int ref_sizeof_config() { return (int)sizeof(Config); }

void *ref_open(const char *ckpt) {
  Transformer *t = (Transformer *)calloc(1, sizeof(Transformer));
  build_transformer(t, (char *)ckpt);
  return t;
}

void ref_close(void *h) {
  Transformer *t = (Transformer *)h;
  free_transformer(t);
  free(t);
}

// logits of one forward() call; the state (KV cache) lives in the handle
const float *ref_forward(void *h, int token, int pos) {
  return forward((Transformer *)h, token, pos);
}

// residual stream after the final norm of the last ref_forward call
const float *ref_state_x(void *h) { return ((Transformer *)h)->state.x; }

int ref_argmax(const float *v, int n) { return sample_argmax((float *)v, n); }

void ref_rope(int pos, float theta, int head_dim, float scaling, float init_ctx, float *cos_out,
              float *sin_out) {
  compute_cos_sin(pos, theta, head_dim, scaling, init_ctx, 32.0f, 1.0f, cos_out, sin_out);
}

void ref_topk(float *vals, int *idx, float *scores, int n_experts, int k) {
  topk(vals, idx, scores, n_experts, k);
  softmax(vals, k);
}

long long ref_generate(const char *ckpt, const int *prompts, const int *n_prompt,
                       int prompt_stride, int n_req, int max_seq_len, int *out) {
  long long total = 0;
  for (int r = 0; r < n_req; r++) {
    Transformer t;
    build_transformer(&t, (char *)ckpt);
    const int *pt = prompts + (long long)r * prompt_stride;
    int *o = out + (long long)r * (max_seq_len + 1);
    int np = n_prompt[r];
    int token = pt[0];
    int cur = 0;
    for (int pos = 0; pos < max_seq_len - 1; pos++) {
      float *logits = forward(&t, token, pos);
      int next = sample_argmax(logits, t.config.vocab_size);
      if (cur < np - 1) {
        next = pt[cur + 1];
      } else {
        o[cur - (np - 1)] = next;
      }
      token = next;
      cur++;
      if (next == 199999 || next == 200002) break;
    }
    int generated_len = cur - np;
    if (generated_len < 0) generated_len = 0;
    o[generated_len + 1] = -1;
    total += generated_len + 1;
    free_transformer(&t);
  }
  return total;
}

}  // extern "C"
