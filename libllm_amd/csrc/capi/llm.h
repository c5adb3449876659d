/* C API of libllm_amd, with the names and the manner of the reference's (src/libllm/llm.h:42-72):
 * every argument and result is a JSON object, a call returns 0 or an error code, and the message
 * of the last error of the calling thread is kept.  The library runs the Python package
 * libllm_amd inside the process (it starts an interpreter if none is running).
 *
 *   llm_json_t kwargs, chunk;  llm_model_t model;  llm_completion_t comp;
 *   llm_init();
 *   llm_json_init(&kwargs);  llm_json_parse(&kwargs, "{\"filename\": \"DIR\", \"device\": \"auto\"}");
 *   llm_model_init(&model);  llm_model_load(&model, &kwargs);
 *   llm_json_parse(&kwargs, "{\"token_ids\": [1, 2, 3], \"temperature\": 1.0, \"top_k\": 1}");
 *   llm_completion_init(&comp);  llm_model_complete(&model, &kwargs, &comp);
 *   llm_json_init(&chunk);
 *   while (llm_completion_get_next_chunk(&comp, &chunk) == 0) { llm_json_dump(&chunk, buf, sizeof buf); ... }
 */
#ifndef LIBLLM_AMD_LLM_H_
#define LIBLLM_AMD_LLM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLM_ERROR_INVALID_ARG 0x0100
#define LLM_ERROR_INSUFFICIENT_BUFFER 0x0101
#define LLM_ERROR_ABORTED 0x0102
#define LLM_ERROR_EOF 0x0103

typedef struct llm_model_impl_t *llm_model_t;
typedef struct llm_completion_impl_t *llm_completion_t;
typedef struct llm_json_impl_t *llm_json_t;

/* global state */
void llm_init(void);
const char *llm_get_last_error_message(void);

/* JSON */
int32_t llm_json_init(llm_json_t *j);
int32_t llm_json_destroy(llm_json_t *j);
int32_t llm_json_parse(llm_json_t *j, const char *json_str);
int32_t llm_json_dump(llm_json_t *j, char *buf, int64_t buf_size);

/* model: kwargs of load {"filename", "device"} (ours: "dtype", "max_tokens", "max_batch",
 * "random_weights", "seed");
 * info {"name", ...}; kwargs of complete {"messages" or "token_ids", "temperature", "top_k",
 * "top_p"} (ours: "max_new_tokens", "seed") */
int32_t llm_model_init(llm_model_t *m);
int32_t llm_model_destroy(llm_model_t *m);
int32_t llm_model_load(llm_model_t *m, llm_json_t *kwargs);
int32_t llm_model_get_info(llm_model_t *m, llm_json_t *info);
int32_t llm_model_complete(llm_model_t *m, llm_json_t *kwargs, llm_completion_t *comp);

/* Two calls without a counterpart in the reference's C API, for what this library has beside
 * single completions.
 * generate: batches of prompts of token ids, unequal lengths, as many batches as the cache needs:
 *   kwargs {"prompts": [[1, 2, 3], [4, 5]], "max_new_tokens", "temperature", "top_k", "top_p",
 *   "seed", "stop_tokens"}; result {"tokens": [[...], [...]]}.
 * step: one call of the step function, in the words of a line of a trace:
 *   kwargs {"entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []};
 *   the float32 logits at the wanted places, [wanted, vocab] (vocab_size of get_info), go to
 *   `logits`, which holds `capacity` floats; *n_rows is the number of wanted rows.  If they do not
 *   fit, nothing runs, *n_rows is the number of floats needed and LLM_ERROR_INSUFFICIENT_BUFFER is
 *   returned. */
int32_t llm_model_generate(llm_model_t *m, llm_json_t *kwargs, llm_json_t *result);
int32_t llm_model_step(llm_model_t *m, llm_json_t *kwargs, float *logits, int64_t capacity, int64_t *n_rows);

/* completion: chunk {"text", "token_id"}; LLM_ERROR_EOF after the last one */
int32_t llm_completion_init(llm_completion_t *c);
int32_t llm_completion_destroy(llm_completion_t *c);
int32_t llm_completion_get_next_chunk(llm_completion_t *c, llm_json_t *chunk);

#ifdef __cplusplus
}
#endif

#endif  /* LIBLLM_AMD_LLM_H_ */
