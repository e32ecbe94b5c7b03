/* Failure handling of the C interface, no GPU needed: statuses, messages, the error slot. */
#include <stdio.h>
#include <string.h>

#include "sonicboom_amd.h"

#define CHECK(cond)                                           \
  do {                                                        \
    if (!(cond)) {                                            \
      printf("FAILED line %d: %s\n", __LINE__, #cond);        \
      return 1;                                               \
    }                                                         \
  } while (0)

int main(void) {
  boom_error *err = NULL;
  boom_llm_model *model = (boom_llm_model *)0x1;
  boom_status st = boom_llm_model_load("/nonexistent/folder", NULL, &model, &err);
  CHECK(st == BOOM_ERR_CONFIG);
  CHECK(model == NULL);
  CHECK(err != NULL && strstr(boom_error_message(err), "config.json") != NULL);
  /* the slot is reused: the old handle is released, a new one written */
  st = boom_llm_model_load(NULL, NULL, &model, &err);
  CHECK(st == BOOM_ERR_INTERNAL);
  CHECK(strstr(boom_error_message(err), "NULL") != NULL);
  /* no slot: only the status */
  CHECK(boom_llm_model_random("/nonexistent/config.json", 1, NULL, &model, NULL) != BOOM_OK);
  /* handles that are not handles */
  size_t n = 0;
  CHECK(boom_llm_model_arch(NULL, NULL, 0, &n, &err) == BOOM_ERR_INTERNAL);
  CHECK(boom_llm_session_new(NULL, 64, NULL, &err) == BOOM_ERR_INTERNAL);
  CHECK(boom_llm_step(NULL, NULL, 0, NULL, 0, &n, &err) == BOOM_ERR_INTERNAL);
  /* pointers that were never handed out are refused without being read */
  {
    uint32_t vocab = 0;
    int32_t slot = 0;
    CHECK(boom_llm_model_vocab((const boom_llm_model *)(uintptr_t)0x10, &vocab, &err) == BOOM_ERR_INTERNAL);
    CHECK(boom_llm_slot_alloc((boom_llm_session *)(uintptr_t)0x10, &slot, &err) == BOOM_ERR_INTERNAL);
    boom_llm_model_free((boom_llm_model *)(uintptr_t)0x10);
    boom_llm_session_free((boom_llm_session *)(uintptr_t)0x10);
  }
  boom_llm_model_free(NULL);
  boom_llm_session_free(NULL);
  CHECK(strcmp(boom_error_message(NULL), "") == 0);
  boom_error_free(err);
  CHECK(strstr(boom_build_info(), "sonicboom_amd") != NULL);
  printf("ok\n");
  return 0;
}
