/* Walks the C interface on a model folder (argv[1], dtype argv[2]): queries, one step, a batch
 * generation with a callback that cuts one prompt short (the refused token is not reported).
 * Prints what it got, one item a line, for the Python test to compare with the package's own
 * results. */
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "sonicboom_amd.h"

#define MUST(call)                                                        \
  do {                                                                    \
    if ((call) != BOOM_OK) {                                              \
      printf("FAILED line %d: %s\n", __LINE__, boom_error_message(err));  \
      return 1;                                                           \
    }                                                                     \
  } while (0)

static int stop_second_prompt_at_its_third_token(void *user, uint32_t prompt, boom_token token) {
  int *seen = (int *)user;
  (void)token;
  if (prompt == 1) return ++*seen >= 3;
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 3) return 2;
  boom_error *err = NULL;
  boom_llm_load_options lo;
  memset(&lo, 0, sizeof lo);
  lo.struct_size = sizeof lo;
  lo.dtype = argv[2];
  boom_llm_model *model = NULL;
  MUST(boom_llm_model_load(argv[1], &lo, &model, &err));

  size_t n = 0;
  if (boom_llm_model_arch(model, NULL, 0, &n, &err) != BOOM_ERR_BINDING) return 3;   /* sizing call */
  char *arch = (char *)malloc(n);
  MUST(boom_llm_model_arch(model, arch, n, &n, &err));
  printf("arch %s\n", arch);
  uint32_t vocab = 0;
  MUST(boom_llm_model_vocab(model, &vocab, &err));
  printf("vocab %u\n", vocab);
  boom_token eos[16];
  size_t n_eos = 0;
  MUST(boom_llm_model_eos(model, eos, 16, &n_eos, &err));
  printf("eos");
  for (size_t i = 0; i < n_eos; ++i) printf(" %d", eos[i]);
  printf("\n");

  boom_llm_session *session = NULL;
  MUST(boom_llm_session_new(model, 512, &session, &err));
  /* the session keeps its model alive: the model handle is given back before any step */
  boom_llm_model_free(model);
  if (boom_llm_model_vocab(model, &vocab, &err) != BOOM_ERR_INTERNAL) return 7;   /* a freed handle is refused */
  boom_llm_model_free(model);                                                      /* twice: ignored */

  /* one step: two sequences of unequal length, logits at three places */
  int32_t s0 = -1, s1 = -1;
  MUST(boom_llm_slot_alloc(session, &s0, &err));
  MUST(boom_llm_slot_alloc(session, &s1, &err));
  const boom_token t0[] = {5, 17, 3, 9, 250}, t1[] = {7, 7};
  const uint32_t w0[] = {0, 4}, w1[] = {1};
  boom_llm_step_entry entries[2] = {{s0, t0, 5, w0, 2}, {s1, t1, 2, w1, 1}};
  size_t need = 0;
  if (boom_llm_step(session, entries, 2, NULL, 0, &need, &err) != BOOM_ERR_BINDING) return 4;   /* sizing call */
  if (need != 3u * vocab) return 5;
  float *logits = (float *)malloc(need * sizeof(float));
  MUST(boom_llm_step(session, entries, 2, logits, need, &need, &err));
  for (int r = 0; r < 3; ++r) {
    int best = 0;
    for (uint32_t v = 1; v < vocab; ++v)
      if (logits[r * vocab + v] > logits[r * vocab + best]) best = (int)v;
    printf("step row %d argmax %d logit %.6f\n", r, best, logits[r * vocab + best]);
  }
  MUST(boom_llm_slot_free(session, s0, &err));
  MUST(boom_llm_slot_free(session, s1, &err));
  if (boom_llm_slot_free(session, s1, &err) == BOOM_OK) return 6;      /* freed twice: refused */

  /* generation: three prompts, greedy, the callback refuses the second one's third token */
  const boom_token p0[] = {1, 2, 3}, p1[] = {4, 5, 6, 7, 8, 9, 10}, p2[] = {11};
  const boom_token *prompts[3] = {p0, p1, p2};
  const size_t lens[3] = {3, 7, 1};
  boom_llm_sampling sp;
  memset(&sp, 0, sizeof sp);
  sp.struct_size = sizeof sp;
  sp.max_tokens = 6;
  const boom_token no_stop[1] = {-1};
  boom_token out[18];
  uint32_t counts[3];
  int seen = 0;
  MUST(boom_llm_generate(session, prompts, lens, 3, &sp, no_stop, 0, stop_second_prompt_at_its_third_token, &seen, out, counts,
                         &err));
  for (int i = 0; i < 3; ++i) {
    printf("greedy %d:", i);
    for (uint32_t j = 0; j < counts[i]; ++j) printf(" %d", out[i * 6 + j]);
    printf("\n");
  }
  /* a penalty with an explicit empty window penalises nothing; a struct that ends before
   * repeat_last_n gets the window of 64 and does */
  sp.repeat_penalty = 5.0f;
  sp.repeat_last_n = 0;
  boom_token out2[18];
  uint32_t counts2[3];
  MUST(boom_llm_generate(session, prompts, lens, 3, &sp, no_stop, 0, NULL, NULL, out2, counts2, &err));
  printf("empty window %s\n", (counts2[0] == 6 && memcmp(out2, out, 6 * sizeof(boom_token)) == 0) ? "same" : "differs");
  sp.struct_size = offsetof(boom_llm_sampling, repeat_last_n);
  sp.repeat_last_n = 12345;                     /* not read: beyond struct_size */
  MUST(boom_llm_generate(session, prompts, lens, 3, &sp, no_stop, 0, NULL, NULL, out2, counts2, &err));
  printf("short struct:");
  for (uint32_t j = 0; j < counts2[0]; ++j) printf(" %d", out2[j]);
  printf("\n");
  sp.struct_size = sizeof sp;
  sp.repeat_penalty = 0.0f;
  sp.repeat_last_n = 0;
  /* sampled, seeded */
  sp.temperature = 0.8f;
  sp.seed = 7;
  sp.top_k = 40;
  MUST(boom_llm_generate(session, prompts, lens, 3, &sp, no_stop, 0, NULL, NULL, out, counts, &err));
  for (int i = 0; i < 3; ++i) {
    printf("sampled %d:", i);
    for (uint32_t j = 0; j < counts[i]; ++j) printf(" %d", out[i * 6 + j]);
    printf("\n");
  }
  /* prefix reuse: a conversation that goes on feeds only what is new, and says the same */
  sp.temperature = 0.0f;
  sp.top_k = 0;
  sp.max_tokens = 4;
  MUST(boom_llm_session_keep(session, 1, &err));
  boom_token first[4];
  uint32_t n_first = 0;
  const boom_token *one[1] = {p1};
  const size_t one_len[1] = {7};
  MUST(boom_llm_generate(session, one, one_len, 1, &sp, no_stop, 0, NULL, NULL, first, &n_first, &err));
  boom_token longer[7 + 3 + 2] = {4, 5, 6, 7, 8, 9, 10, 0, 0, 0, 33, 34};
  for (int j = 0; j < 3; ++j) longer[7 + j] = first[j];
  const boom_token *two[1] = {longer};
  const size_t two_len[1] = {12};
  boom_token second[4];
  uint32_t n_second = 0;
  MUST(boom_llm_generate(session, two, two_len, 1, &sp, no_stop, 0, NULL, NULL, second, &n_second, &err));
  uint64_t reused[1] = {0};
  size_t n_reused = 0;
  if (boom_llm_session_reused(session, NULL, 0, &n_reused, &err) != BOOM_ERR_BINDING || n_reused != 1) return 9;
  MUST(boom_llm_session_reused(session, reused, 1, &n_reused, &err));
  printf("reused %llu:", (unsigned long long)reused[0]);
  for (uint32_t j = 0; j < n_second; ++j) printf(" %d", second[j]);
  printf("\n");
  MUST(boom_llm_session_keep(session, 0, &err));
  free(logits);
  free(arch);
  boom_llm_session_free(session);
  if (boom_llm_slot_alloc(session, &s0, &err) != BOOM_ERR_INTERNAL) return 8;      /* a freed session is refused */
  boom_llm_session_free(session);
  boom_error_free(err);
  printf("ok\n");
  return 0;
}
