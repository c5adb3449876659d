// The `llm` program over the C API (llm.h), as the reference's command line is a program over its
// C API (go/bin/main.go:27-54, go/bin/args.go:54-91, go/bin/chat.go:44-132):
//
//   llm chat -m MODEL [-device cpu|cuda|hip|auto] [-dtype bfloat16|float32] [-max_tokens N]
//            [-temperature T] [-top_k K] [-top_p P] [-seed S] [-max_new_tokens N] [-ids]
//            [-random_weights] [-stop_id ID]...
//
// A prompt loop with `:new` (clear the history), `:sys <prompt>` (set the system prompt and clear),
// empty lines ignored, end of input leaving; after each reply `(N tokens, time=..s, ..ms per token)`.
// Flags take one or two dashes.  With -ids a line is a list of token ids and the reply is printed
// as ids.  The messages and their order are those of the Python command line (libllm_amd/cli.py).
#include <cctype>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <sstream>
#include <string>
#include <utility>
#include <vector>

#include "llm.h"

namespace {

const char *kInput = "Please input your question.";
const char *kNew = "    Type ':new' to start a new session (clean history).";
const char *kSys = "    Type ':sys <system_prompt>' to set the system prompt and start a new session .";
const char *kNewSession = "===== new session =====";

void usage() {
  std::fprintf(stderr,
               "Usage: llm COMMAND\n\nCommands:\n    chat           Chat with LLM\n\n"
               "Run 'llm COMMAND -h' for more information on a command.\n");
}

void chat_usage() {
  std::fprintf(stderr,
               "usage: llm chat -m MODEL [-device DEVICE] [-dtype {bfloat16,float32}] [-max_tokens N]\n"
               "                [-temperature T] [-top_k K] [-top_p P] [-seed S] [-max_new_tokens N] [-ids]\n"
               "                [-random_weights] [-stop_id ID]...\n");
}

[[noreturn]] void arg_error(const std::string &msg) {
  chat_usage();
  std::fprintf(stderr, "llm chat: error: %s\n", msg.c_str());
  std::exit(2);
}

// text as a JSON string literal
std::string quoted(const std::string &s) {
  std::string out = "\"";
  char buf[8];
  for (unsigned char c : s) {
    if (c == '"') out += "\\\"";
    else if (c == '\\') out += "\\\\";
    else if (c == '\n') out += "\\n";
    else if (c == '\r') out += "\\r";
    else if (c == '\t') out += "\\t";
    else if (c < 0x20) { std::snprintf(buf, sizeof buf, "\\u%04x", c); out += buf; }
    else out += (char)c;
  }
  return out + "\"";
}

void append_utf8(std::string &out, uint32_t cp) {
  if (cp < 0x80) out += (char)cp;
  else if (cp < 0x800) { out += (char)(0xc0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3f)); }
  else if (cp < 0x10000) {
    out += (char)(0xe0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3f)); out += (char)(0x80 | (cp & 0x3f));
  } else {
    out += (char)(0xf0 | (cp >> 18)); out += (char)(0x80 | ((cp >> 12) & 0x3f));
    out += (char)(0x80 | ((cp >> 6) & 0x3f)); out += (char)(0x80 | (cp & 0x3f));
  }
}

// The JSON string literal that starts at text[pos] (a quote); pos moves past it.
bool read_string(const std::string &text, size_t &pos, std::string &out) {
  if (pos >= text.size() || text[pos] != '"') return false;
  out.clear();
  for (++pos; pos < text.size(); ++pos) {
    const char c = text[pos];
    if (c == '"') { ++pos; return true; }
    if (c != '\\') { out += c; continue; }
    if (++pos >= text.size()) return false;
    switch (text[pos]) {
      case 'n': out += '\n'; break;
      case 't': out += '\t'; break;
      case 'r': out += '\r'; break;
      case 'b': out += '\b'; break;
      case 'f': out += '\f'; break;
      case 'u': {
        if (pos + 4 >= text.size()) return false;
        uint32_t cp = (uint32_t)std::strtoul(text.substr(pos + 1, 4).c_str(), nullptr, 16);
        pos += 4;
        if (cp >= 0xd800 && cp < 0xdc00 && pos + 6 < text.size() && text[pos + 1] == '\\' && text[pos + 2] == 'u') {
          const uint32_t lo = (uint32_t)std::strtoul(text.substr(pos + 3, 4).c_str(), nullptr, 16);
          if (lo >= 0xdc00 && lo < 0xe000) {
            cp = 0x10000 + ((cp - 0xd800) << 10) + (lo - 0xdc00);
            pos += 6;
          }
        }
        append_utf8(out, cp);
        break;
      }
      default: out += text[pos];          // \" \\ \/
    }
  }
  return false;
}

// A chunk as the library dumps it: {"text": "...", "token_id": N or null}.
bool read_chunk(const std::string &json, std::string &text, bool &has_id, long &id) {
  size_t pos = json.find("\"text\":");
  if (pos == std::string::npos) return false;
  pos = json.find('"', pos + 7);
  if (pos == std::string::npos || !read_string(json, pos, text)) return false;
  pos = json.find("\"token_id\":", pos);
  has_id = false;
  if (pos != std::string::npos) {
    const char *p = json.c_str() + pos + 11;
    while (*p == ' ') ++p;
    if (*p == '-' || (*p >= '0' && *p <= '9')) { has_id = true; id = std::strtol(p, nullptr, 10); }
  }
  return true;
}

std::string strip(const std::string &s) {
  size_t a = 0, b = s.size();
  while (a < b && std::isspace((unsigned char)s[a])) ++a;
  while (b > a && std::isspace((unsigned char)s[b - 1])) --b;
  return s.substr(a, b - a);
}

std::string lower(std::string s) {
  for (char &c : s) c = (char)std::tolower((unsigned char)c);
  return s;
}

#define CHECK(call)                                                        \
  do {                                                                     \
    if ((call) != 0) {                                                     \
      std::fprintf(stderr, "llm: %s\n", llm_get_last_error_message());     \
      return 1;                                                            \
    }                                                                      \
  } while (0)

int chat_main(int argc, char **argv) {
  std::vector<std::string> models;
  std::string device = "auto", dtype = "bfloat16";
  long max_tokens = 8192, top_k = 50, seed = 0, max_new = 256;
  double temperature = 1.0, top_p = 0.8;
  bool ids = false, random_weights = false;
  std::vector<long> stop_ids;
  for (int i = 0; i < argc; ++i) {
    std::string flag = argv[i];
    if (flag.size() < 2 || flag[0] != '-') arg_error("unrecognized arguments: " + flag);
    flag = flag.substr(flag[1] == '-' ? 2 : 1);
    for (char &c : flag) if (c == '-') c = '_';
    if (flag == "h" || flag == "help") { chat_usage(); return 0; }
    if (flag == "ids") { ids = true; continue; }
    if (flag == "random_weights") { random_weights = true; continue; }
    if (i + 1 >= argc) arg_error("argument -" + flag + ": expected one argument");
    const std::string value = argv[++i];
    char *end = nullptr;
    auto as_long = [&]() { long v = std::strtol(value.c_str(), &end, 10); if (*end || value.empty()) arg_error("argument -" + flag + ": invalid int value: '" + value + "'"); return v; };
    auto as_double = [&]() { double v = std::strtod(value.c_str(), &end); if (*end || value.empty()) arg_error("argument -" + flag + ": invalid float value: '" + value + "'"); return v; };
    if (flag == "m") models.push_back(value);
    else if (flag == "device") device = lower(value);
    else if (flag == "dtype") dtype = value;
    else if (flag == "max_tokens") max_tokens = as_long();
    else if (flag == "temperature") temperature = as_double();
    else if (flag == "top_k") top_k = as_long();
    else if (flag == "top_p") top_p = as_double();
    else if (flag == "seed") seed = as_long();
    else if (flag == "max_new_tokens") max_new = as_long();
    else if (flag == "stop_id") stop_ids.push_back(as_long());
    else arg_error("unrecognized arguments: -" + flag);
  }
  if (device != "cpu" && device != "cuda" && device != "hip" && device != "auto")
    arg_error("invalid device name: must be one of \"cpu\", \"cuda\" or \"auto\"");
  if (dtype != "bfloat16" && dtype != "float32" && dtype != "bf16" && dtype != "fp32") arg_error("argument -dtype: invalid choice: '" + dtype + "'");
  if (models.empty()) arg_error("model name (-m) is empty.");
  if (models.size() != 1) arg_error("only 1 model (-m) is expected");

  llm_init();
  llm_json_t kwargs, chunk;
  llm_model_t model;
  llm_completion_t comp;
  CHECK(llm_json_init(&kwargs));
  CHECK(llm_json_init(&chunk));
  CHECK(llm_model_init(&model));
  CHECK(llm_completion_init(&comp));
  {
    std::ostringstream js;
    js << "{\"filename\": " << quoted(models[0]) << ", \"device\": " << quoted(device) << ", \"dtype\": "
       << quoted(dtype) << ", \"max_tokens\": " << max_tokens << ", \"random_weights\": "
       << (random_weights ? "true" : "false") << ", \"seed\": " << seed << "}";
    CHECK(llm_json_parse(&kwargs, js.str().c_str()));
    CHECK(llm_model_load(&model, &kwargs));
  }
  std::printf("%s\n%s\n%s\n", kInput, kNew, kSys);

  std::vector<long> id_history;                                    // with -ids
  std::vector<std::pair<std::string, std::string>> history;        // (role, text) otherwise
  std::string system_prompt, line;
  std::vector<char> buf(1 << 20);
  long turn = 0;
  for (;;) {
    std::printf("> ");
    std::fflush(stdout);
    if (!std::getline(std::cin, line)) {
      std::printf("\n");
      break;
    }
    const std::string question = strip(line);
    if (question.size() > 5 && lower(question.substr(0, 5)) == ":sys ") {
      system_prompt = strip(question.substr(5));
      history.clear();
      id_history.clear();
      continue;
    }
    if (lower(question) == ":new") {
      std::printf("%s\n", kNewSession);
      history.clear();
      id_history.clear();
      continue;
    }
    if (question.empty()) continue;

    std::ostringstream js;
    std::vector<long> prompt_ids;
    if (ids) {
      std::string spaced = question;
      for (char &c : spaced) if (c == ',') c = ' ';
      std::istringstream in(spaced);
      std::string tok;
      bool ok = true;
      prompt_ids = id_history;
      while (in >> tok) {
        char *end = nullptr;
        const long v = std::strtol(tok.c_str(), &end, 10);
        if (*end) { ok = false; break; }
        prompt_ids.push_back(v);
      }
      if (!ok) {
        std::printf("with -ids a line must hold token ids\n");
        continue;
      }
      js << "{\"token_ids\": [";
      for (size_t i = 0; i < prompt_ids.size(); ++i) js << (i ? ", " : "") << prompt_ids[i];
      js << "]";
    } else {
      if (history.empty() && !system_prompt.empty()) history.emplace_back("system", system_prompt);
      history.emplace_back("user", question);
      js << "{\"messages\": [";
      for (size_t i = 0; i < history.size(); ++i)
        js << (i ? ", " : "") << "{\"role\": " << quoted(history[i].first) << ", \"content\": "
           << quoted(history[i].second) << "}";
      js << "]";
    }
    js.precision(17);
    js << ", \"temperature\": " << temperature << ", \"top_k\": " << top_k << ", \"top_p\": " << top_p
       << ", \"max_new_tokens\": " << max_new << ", \"seed\": " << (seed + turn);
    if (!stop_ids.empty()) {
      js << ", \"stop_ids\": [";
      for (size_t i = 0; i < stop_ids.size(); ++i) js << (i ? ", " : "") << stop_ids[i];
      js << "]";
    }
    js << "}";
    CHECK(llm_json_parse(&kwargs, js.str().c_str()));

    const auto t0 = std::chrono::steady_clock::now();
    CHECK(llm_model_complete(&model, &kwargs, &comp));
    long n = 0;
    std::string reply_text, text;
    std::vector<long> reply_ids;
    int32_t rc;
    while ((rc = llm_completion_get_next_chunk(&comp, &chunk)) == 0) {
      CHECK(llm_json_dump(&chunk, buf.data(), (int64_t)buf.size()));
      bool has_id = false;
      long id = 0;
      if (!read_chunk(buf.data(), text, has_id, id)) {
        std::fprintf(stderr, "llm: a chunk that cannot be read: %s\n", buf.data());
        return 1;
      }
      if (has_id) {
        ++n;
        reply_ids.push_back(id);
      }
      if (ids) {
        if (has_id) std::printf("%ld ", id);
      } else {
        reply_text += text;
        std::fwrite(text.data(), 1, text.size(), stdout);
      }
      std::fflush(stdout);
    }
    if (rc != LLM_ERROR_EOF) {
      std::fprintf(stderr, "llm: %s\n", llm_get_last_error_message());
      return 1;
    }
    std::printf("\n");
    if (ids) {
      id_history = prompt_ids;
      id_history.insert(id_history.end(), reply_ids.begin(), reply_ids.end());
    } else {
      history.emplace_back("assistant", reply_text);
    }
    const double dur = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("(%ld tokens, time=%.2fs, %.2fms per token)\n", n, dur, dur * 1000.0 / (n > 0 ? n : 1));
    ++turn;
  }
  llm_completion_destroy(&comp);
  llm_model_destroy(&model);
  llm_json_destroy(&kwargs);
  llm_json_destroy(&chunk);
  return 0;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc < 2) {
    usage();
    return 1;
  }
  const std::string command = argv[1];
  if (command == "chat") return chat_main(argc - 2, argv + 2);
  std::fprintf(stderr, "Invalid command \"%s\"\n\n", command.c_str());
  usage();
  return 1;
}
