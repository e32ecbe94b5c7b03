// sb-gen: token ids in, token ids out, over the C interface (sonicboom_amd.h).
//
// In the manner of the reference's token tool (/root/reference/tools/baseline/gen_from_tokens.cpp:
// 34-50 a plain argv loop with -m, --tokens, -n, --ctx; usage on stderr and exit status 2;
// 92-96 one line of produced ids per prompt); the sampling options carry the names of the
// fields of boom_llm_sampling.  The tokens file holds one prompt per line, ids separated by
// blanks.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "sonicboom_amd.h"

namespace {

const char *kUsage =
    "usage: sb-gen (-m MODEL_DIR | --random CONFIG.json [--seed S]) --tokens FILE [-n N] [--ctx N]\n"
    "              [--dtype bfloat16|float32] [--temperature T] [--top-k K] [--top-p P] [--min-p P]\n"
    "              [--sample-seed S] [--repeat-penalty R] [--repeat-last-n N] [--presence-penalty X]\n"
    "              [--frequency-penalty X] [--stop ID,ID,...]\n";

int usage(const char *why) {
  std::fprintf(stderr, "sb-gen: %s\n%s", why, kUsage);
  return 2;
}

int die(const char *what, boom_error *err) {
  std::fprintf(stderr, "sb-gen: %s: %s\n", what, boom_error_message(err));
  boom_error_free(err);
  return 1;
}

}  // namespace

int main(int argc, char **argv) {
  std::string model_dir, random_cfg, tokens_path, dtype = "bfloat16", stop_arg;
  unsigned long long seed = 0, ctx = 0;
  bool have_stop = false;
  boom_llm_sampling sp;
  std::memset(&sp, 0, sizeof sp);
  sp.struct_size = sizeof sp;
  sp.max_tokens = 16;
  sp.top_p = 1.f;
  sp.repeat_penalty = 1.f;
  sp.repeat_last_n = 64;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto value = [&]() -> const char * { return i + 1 < argc ? argv[++i] : nullptr; };
    const char *v = nullptr;
    if (a == "-h" || a == "--help") { std::fputs(kUsage, stdout); return 0; }
#define SB_OPT(flag, stmt) else if (a == flag) { if (!(v = value())) return usage(flag " needs a value"); stmt; }
    SB_OPT("-m", model_dir = v) SB_OPT("--model", model_dir = v) SB_OPT("--random", random_cfg = v)
    SB_OPT("--seed", seed = std::strtoull(v, nullptr, 10)) SB_OPT("--dtype", dtype = v)
    SB_OPT("--tokens", tokens_path = v) SB_OPT("-n", sp.max_tokens = (uint32_t)std::strtoul(v, nullptr, 10))
    SB_OPT("--ctx", ctx = std::strtoull(v, nullptr, 10)) SB_OPT("--temperature", sp.temperature = std::strtof(v, nullptr))
    SB_OPT("--top-k", sp.top_k = (uint32_t)std::strtoul(v, nullptr, 10)) SB_OPT("--top-p", sp.top_p = std::strtof(v, nullptr))
    SB_OPT("--min-p", sp.min_p = std::strtof(v, nullptr)) SB_OPT("--sample-seed", sp.seed = std::strtoull(v, nullptr, 10))
    SB_OPT("--repeat-penalty", sp.repeat_penalty = std::strtof(v, nullptr))
    SB_OPT("--repeat-last-n", sp.repeat_last_n = (uint32_t)std::strtoul(v, nullptr, 10))
    SB_OPT("--presence-penalty", sp.presence_penalty = std::strtof(v, nullptr))
    SB_OPT("--frequency-penalty", sp.frequency_penalty = std::strtof(v, nullptr))
    SB_OPT("--stop", (stop_arg = v, have_stop = true))
#undef SB_OPT
    else return usage(("unknown option " + a).c_str());
  }
  if (model_dir.empty() == random_cfg.empty()) return usage("give exactly one of -m and --random");
  if (tokens_path.empty()) return usage("--tokens is required");
  if (dtype == "bf16") dtype = "bfloat16";
  if (dtype == "fp32") dtype = "float32";
  if (dtype != "bfloat16" && dtype != "float32") return usage("--dtype is bfloat16 or float32");

  std::ifstream in(tokens_path);
  if (!in) {
    std::fprintf(stderr, "tokens file not found: %s\n", tokens_path.c_str());
    return 2;
  }
  std::vector<std::vector<boom_token>> prompts;
  for (std::string line; std::getline(in, line);) {
    std::istringstream ls(line);
    std::vector<boom_token> ids;
    for (long long t; ls >> t;) ids.push_back((boom_token)t);
    if (!ls.eof()) return usage("the tokens file holds something that is not a token id");
    if (!ids.empty()) prompts.push_back(ids);
  }
  if (prompts.empty()) return usage("the tokens file holds no prompt");
  std::vector<boom_token> stops;
  if (have_stop) {
    std::istringstream ss(stop_arg);
    for (std::string item; std::getline(ss, item, ',');)
      if (!item.empty()) stops.push_back((boom_token)std::strtol(item.c_str(), nullptr, 10));
  }

  boom_llm_load_options lo;
  std::memset(&lo, 0, sizeof lo);
  lo.struct_size = sizeof lo;
  lo.dtype = dtype.c_str();
  boom_error *err = nullptr;
  boom_llm_model *model = nullptr;
  const boom_status st = model_dir.empty() ? boom_llm_model_random(random_cfg.c_str(), seed, &lo, &model, &err)
                                           : boom_llm_model_load(model_dir.c_str(), &lo, &model, &err);
  if (st != BOOM_OK) return die("cannot load the model", err);
  if (ctx == 0)   // what the prompts need, each sequence rounded up to the cache's pages of 64
    for (const auto &p : prompts) ctx += (p.size() + sp.max_tokens + 63) / 64 * 64;
  boom_llm_session *session = nullptr;
  if (boom_llm_session_new(model, ctx, &session, &err) != BOOM_OK) return die("cannot make a session", err);

  std::vector<const boom_token *> rows;
  std::vector<size_t> lens;
  for (const auto &p : prompts) {
    rows.push_back(p.data());
    lens.push_back(p.size());
  }
  std::vector<boom_token> out(prompts.size() * (size_t)sp.max_tokens + 1);
  std::vector<uint32_t> counts(prompts.size());
  if (boom_llm_generate(session, rows.data(), lens.data(), prompts.size(), &sp, have_stop ? stops.data() : nullptr,
                        stops.size(), nullptr, nullptr, out.data(), counts.data(), &err) != BOOM_OK)
    return die("generation failed", err);
  for (size_t i = 0; i < prompts.size(); ++i) {
    for (uint32_t j = 0; j < counts[i]; ++j) std::printf(j ? " %d" : "%d", out[i * sp.max_tokens + j]);
    std::printf("\n");
  }
  boom_llm_session_free(session);
  boom_llm_model_free(model);
  return 0;
}
