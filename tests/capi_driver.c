/* A C program over the C API: loads a model folder, completes one prompt of token ids greedily
 * and prints the token ids of the chunks, one a line.  Usage: capi_driver DIR DTYPE "1, 2, 3" N */
#include <stdio.h>
#include <string.h>

#include "llm.h"

#define CHECK(call)                                                         \
  do {                                                                      \
    int32_t rc_ = (call);                                                   \
    if (rc_ != 0) {                                                         \
      fprintf(stderr, "%s: 0x%x %s\n", #call, rc_, llm_get_last_error_message()); \
      return 1;                                                             \
    }                                                                       \
  } while (0)

int main(int argc, char **argv) {
  if (argc != 5) return 2;
  char text[4096], buf[4096];
  llm_json_t kwargs, chunk, info;
  llm_model_t model;
  llm_completion_t comp;
  llm_init();
  CHECK(llm_json_init(&kwargs));
  CHECK(llm_json_init(&chunk));
  CHECK(llm_json_init(&info));
  snprintf(text, sizeof text, "{\"filename\": \"%s\", \"device\": \"auto\", \"dtype\": \"%s\", \"max_tokens\": 1024}",
           argv[1], argv[2]);
  CHECK(llm_json_parse(&kwargs, text));
  CHECK(llm_model_init(&model));
  CHECK(llm_model_load(&model, &kwargs));
  CHECK(llm_model_get_info(&model, &info));
  CHECK(llm_json_dump(&info, buf, sizeof buf));
  printf("info %s\n", buf);
  snprintf(text, sizeof text, "{\"token_ids\": [%s], \"temperature\": 1.0, \"top_k\": 1, \"max_new_tokens\": %s}",
           argv[3], argv[4]);
  CHECK(llm_json_parse(&kwargs, text));
  CHECK(llm_completion_init(&comp));
  CHECK(llm_model_complete(&model, &kwargs, &comp));
  int32_t rc;
  while ((rc = llm_completion_get_next_chunk(&comp, &chunk)) == 0) {
    CHECK(llm_json_dump(&chunk, buf, sizeof buf));
    printf("chunk %s\n", buf);
  }
  if (rc != LLM_ERROR_EOF) {
    fprintf(stderr, "next_chunk: 0x%x %s\n", rc, llm_get_last_error_message());
    return 1;
  }
  CHECK(llm_completion_destroy(&comp));
  CHECK(llm_model_destroy(&model));
  CHECK(llm_json_destroy(&kwargs));
  CHECK(llm_json_destroy(&chunk));
  CHECK(llm_json_destroy(&info));
  printf("end\n");
  return 0;
}
