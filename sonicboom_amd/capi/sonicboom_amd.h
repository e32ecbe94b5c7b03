/* C interface of sonicboom_amd: load a model folder, make a session (the cache), run steps of a
 * batch of sequences, generate.  Token ids in, token ids out; there is no tokenizer.
 *
 * In the manner of /root/reference/capi/include/sonicboom/capi.h (:42-49 opaque handles,
 * :52-62 status codes, :136-161 error handles, :648-661 option structs that carry their size,
 * :732-735 two-call sizing, :663-682 the sampling options and the token callback): the names of
 * the calls that exist there are kept (boom_llm_model_free, boom_llm_model_arch,
 * boom_llm_model_eos, boom_llm_session_new, boom_llm_session_free, boom_llm_sampling and its
 * fields, boom_error_message, boom_error_free, boom_build_info).  What the reference does not
 * have is the batch: slots, a step over several sequences, generation of several prompts.
 *
 * The library hosts the Python package that composes the model from parts and launches the HIP
 * kernels; a program that is not Python gets an interpreter of its own at the first call.
 * Calls are serialised (one interpreter lock).  No exception crosses this interface: every
 * failure is a status code plus, if the caller passed a slot, an error handle with a message.
 *
 * Error slots: pass NULL, or the address of a boom_error* that is NULL or holds a handle from
 * an earlier call (it is released before a new one is written).  Release the last one with
 * boom_error_free.
 */
#ifndef SONICBOOM_AMD_H
#define SONICBOOM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct boom_llm_model boom_llm_model;     /* weights and parts of one model       */
typedef struct boom_llm_session boom_llm_session; /* a cache and the sequences living in it */
typedef struct boom_error boom_error;             /* a failure's message                  */
typedef int32_t boom_token;                       /* a vocabulary index                   */

typedef enum boom_status {
  BOOM_OK = 0,
  BOOM_ERR_CONFIG = 1,      /* config.json missing, unreadable or refused (the message names the key) */
  BOOM_ERR_WEIGHT = 2,      /* tensors missing, unexpected, ill-shaped or unreadable               */
  BOOM_ERR_BINDING = 4,     /* a buffer too small, an unknown slot, a bad token, no room in the cache */
  BOOM_ERR_RUNTIME = 5,     /* the GPU or the kernel library failed or is absent                   */
  BOOM_ERR_INTERNAL = 6,    /* invalid argument (NULL, freed handle) or an unexpected failure      */
  BOOM_ERR_UNSUPPORTED = 7, /* sizes or options this build does not take                           */
  BOOM_ERR_CANCELLED = 8    /* (reserved) */
} boom_status;

/* Zero the struct, set struct_size = sizeof, then the fields you need. */
typedef struct boom_llm_load_options {
  size_t struct_size;
  const char *dtype;  /* "bfloat16" (default when NULL) or "float32": the true 32-bit path */
  int32_t device;     /* GPU index, default 0 */
} boom_llm_load_options;

/* Same fields and meanings as the reference's struct; 0-initialised = greedy, no filters, and
 * repeat_penalty 0 reads as 1. */
typedef struct boom_llm_sampling {
  size_t struct_size;
  float temperature;       /* 0: greedy (ties to the lower id) */
  float top_p;             /* 0 or 1: off */
  uint32_t top_k;          /* 0: off */
  uint64_t seed;           /* draws are keyed by (seed, absolute position, token id) */
  uint32_t max_tokens;     /* tokens to produce per prompt */
  float min_p;
  float repeat_penalty;
  uint32_t repeat_last_n;  /* window of the penalties; 0: empty, no penalty applies; 64 when struct_size ends before it */
  float presence_penalty;
  float frequency_penalty;
} boom_llm_sampling;

/* One sequence's share of a step: its next tokens and the places among them whose logits are
 * wanted (may be none). */
typedef struct boom_llm_step_entry {
  int32_t slot;
  const boom_token *tokens;
  size_t n_tokens;
  const uint32_t *want;
  size_t n_want;
} boom_llm_step_entry;

/* Called for every produced token of prompt `prompt`; a non-zero return ends that prompt's
 * sequence before that token: it is not reported. */
typedef int (*boom_llm_batch_token_cb)(void *user, uint32_t prompt, boom_token token);

/* --- model ------------------------------------------------------------------------------- */
/* A folder with config.json and model.safetensors (or shards with an index); the model class is
 * chosen by config.json's "architectures". */
boom_status boom_llm_model_load(const char *folder, const boom_llm_load_options *options,
                                boom_llm_model **model_out, boom_error **err_out);
/* Random weights (seeded) for the configuration in a config.json file. */
boom_status boom_llm_model_random(const char *config_json_path, uint64_t seed,
                                  const boom_llm_load_options *options, boom_llm_model **model_out,
                                  boom_error **err_out);
void boom_llm_model_free(boom_llm_model *model);
/* Two-call sizing: with cap too small nothing is written but *len_out / *n_out (BOOM_ERR_BINDING). */
boom_status boom_llm_model_arch(const boom_llm_model *model, char *out, size_t cap, size_t *len_out,
                                boom_error **err_out);
boom_status boom_llm_model_eos(const boom_llm_model *model, boom_token *out, size_t cap, size_t *n_out,
                               boom_error **err_out);
boom_status boom_llm_model_vocab(const boom_llm_model *model, uint32_t *vocab_out, boom_error **err_out);

/* --- session ----------------------------------------------------------------------------- */
/* A cache for at most max_tokens live tokens, each sequence's count rounded up to 64. */
boom_status boom_llm_session_new(boom_llm_model *model, uint64_t max_tokens,
                                 boom_llm_session **session_out, boom_error **err_out);
void boom_llm_session_free(boom_llm_session *session);
boom_status boom_llm_slot_alloc(boom_llm_session *session, int32_t *slot_out, boom_error **err_out);
boom_status boom_llm_slot_free(boom_llm_session *session, int32_t slot, boom_error **err_out);

/* Run the given tokens of every entry as one batch from the cache and write the float32 logits
 * of the wanted places, in the order of the entries and of `want`, [wanted][vocab].  cap counts
 * floats; when it is too small nothing runs, *n_out gets the needed count (BOOM_ERR_BINDING). */
boom_status boom_llm_step(boom_llm_session *session, const boom_llm_step_entry *entries, size_t n_entries,
                          float *logits_out, size_t cap, size_t *n_out, boom_error **err_out);

/* Generate for n_prompts prompts: batches as the cache allows, prompts of a batch in one step,
 * then one token each; a sequence ends at a stop token (which is emitted) or after
 * sampling->max_tokens.  stop == NULL: the model's own eos ids.  out holds
 * n_prompts * sampling->max_tokens tokens (row i = prompt i), n_out[i] the count of row i. */
boom_status boom_llm_generate(boom_llm_session *session, const boom_token *const *prompts,
                              const size_t *prompt_lens, size_t n_prompts,
                              const boom_llm_sampling *sampling, const boom_token *stop, size_t n_stop,
                              boom_llm_batch_token_cb cb, void *user, boom_token *out, uint32_t *n_out,
                              boom_error **err_out);

/* Prefix reuse.  With keep != 0, the sequences of a boom_llm_generate call stay in the cache when
 * they end, and a prompt of the next call that starts with the tokens of one of them feeds only
 * the rest (at most all but its last token are reused); sequences that no prompt of the next call
 * continues are freed when it starts.  keep == 0 (the default) frees what is kept.  The produced
 * tokens do not depend on it. */
boom_status boom_llm_session_keep(boom_llm_session *session, int keep, boom_error **err_out);
/* Per prompt of the last boom_llm_generate call: the tokens that were taken from a kept sequence
 * instead of being fed again.  Two-call sizing as above. */
boom_status boom_llm_session_reused(boom_llm_session *session, uint64_t *out, size_t cap, size_t *n_out,
                                    boom_error **err_out);

/* --- errors, build ----------------------------------------------------------------------- */
const char *boom_error_message(const boom_error *err);  /* never NULL */
void boom_error_free(boom_error *err);
/* A JSON object: package version, kernel libraries and how they were built. Static storage. */
const char *boom_build_info(void);

#ifdef __cplusplus
}
#endif
#endif
