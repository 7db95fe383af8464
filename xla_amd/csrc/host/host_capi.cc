// C entry points of the HLO side of libxla_amd_host.so: parse, run the rewrite pass, print,
// and dump a module as JSON for tools that walk it (the offline module runner).
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>

#include "hlo_ir.h"
#include "quant_fusion_rewriter.h"

#define HOST_EXPORT extern "C" __attribute__((visibility("default")))

namespace {
char* Dup(const std::string& s) {
  char* p = (char*)malloc(s.size() + 1);
  memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

std::string JsonEscape(const std::string& s) {
  std::string o;
  for (char c : s) {
    if (c == '"' || c == '\\') { o += '\\'; o += c; }
    else if (c == '\n') o += "\\n";
    else o += c;
  }
  return o;
}

std::string ShapeJson(const xla_amd::hlo::Shape& s) {
  if (s.is_tuple) {
    std::string o = "{\"tuple\":[";
    for (size_t i = 0; i < s.elements.size(); ++i) o += (i ? "," : "") + ShapeJson(s.elements[i]);
    return o + "]}";
  }
  std::string o = "{\"dtype\":\"" + s.dtype + "\",\"dims\":[";
  for (size_t i = 0; i < s.dims.size(); ++i) o += (i ? "," : "") + std::to_string(s.dims[i]);
  return o + "],\"layout\":\"" + s.layout + "\"}";
}
}  // namespace

struct XlaAmdRewriteCallbacks {
  size_t (*dequant_workspace_bytes)(int64_t, int64_t, int64_t, int64_t, int32_t);
  size_t (*fp8_workspace_bytes)(int64_t, int64_t, int64_t, int32_t, int32_t);
  size_t (*dequant_nk_workspace_bytes)(int64_t, int64_t, int64_t, int64_t, int32_t);
};

// Returns the rewritten module text (malloc'd; free with xla_amd_host_free), or NULL with the
// parse error in *log.  *log (malloc'd) lists one line per rewrite ("rewrite: ...") and per
// refusal ("refused: ..."); *num_rewrites receives the count.
HOST_EXPORT char* xla_amd_hlo_rewrite(const char* text, const XlaAmdRewriteCallbacks* cb, char** log,
                                      int* num_rewrites) {
  std::string err;
  auto mod = xla_amd::hlo::Parse(text, &err);
  if (!mod) {
    if (log) *log = Dup("error: " + err);
    return nullptr;
  }
  xla_amd::hlo::RewriteOptions opt;
  if (cb) {
    opt.dequant_workspace_bytes = cb->dequant_workspace_bytes;
    opt.fp8_workspace_bytes = cb->fp8_workspace_bytes;
    opt.dequant_nk_workspace_bytes = cb->dequant_nk_workspace_bytes;
  }
  xla_amd::hlo::RewriteLog rl;
  int n = xla_amd::hlo::RunQuantFusionRewriter(mod.get(), opt, &rl);
  if (num_rewrites) *num_rewrites = n;
  if (log) {
    std::string l;
    for (auto& r : rl.rewrites) l += "rewrite: " + r + "\n";
    for (auto& r : rl.refusals) l += "refused: " + r + "\n";
    *log = Dup(l);
  }
  return Dup(mod->ToString());
}

// Parses and prints back (round-trip), or NULL with *error set.
HOST_EXPORT char* xla_amd_hlo_print(const char* text, char** error) {
  std::string err;
  auto mod = xla_amd::hlo::Parse(text, &err);
  if (!mod) {
    if (error) *error = Dup(err);
    return nullptr;
  }
  return Dup(mod->ToString());
}

HOST_EXPORT char* xla_amd_hlo_to_json(const char* text, char** error) {
  std::string err;
  auto mod = xla_amd::hlo::Parse(text, &err);
  if (!mod) {
    if (error) *error = Dup(err);
    return nullptr;
  }
  std::string o = "{\"header\":\"" + JsonEscape(mod->header) + "\",\"computations\":[";
  bool firstc = true;
  for (auto& c : mod->computations) {
    o += (firstc ? "" : ",");
    firstc = false;
    o += "{\"name\":\"" + JsonEscape(c->name) + "\",\"entry\":" + (c->is_entry ? "true" : "false") + ",\"instructions\":[";
    const auto* root = c->root();
    bool firsti = true;
    for (auto& i : c->instrs) {
      o += (firsti ? "" : ",");
      firsti = false;
      o += "{\"name\":\"" + JsonEscape(i->name) + "\",\"opcode\":\"" + i->opcode + "\",\"shape\":" + ShapeJson(i->shape) +
           ",\"root\":" + (i.get() == root ? "true" : "false") + ",\"literal\":\"" + JsonEscape(i->literal) + "\",\"operands\":[";
      for (size_t k = 0; k < i->operands.size(); ++k) o += (k ? "," : "") + ("\"" + JsonEscape(i->operands[k]->name) + "\"");
      o += "],\"attrs\":{";
      for (size_t k = 0; k < i->attrs.size(); ++k)
        o += (k ? "," : "") + ("\"" + JsonEscape(i->attrs[k].first) + "\":\"" + JsonEscape(i->attrs[k].second) + "\"");
      o += "}}";
    }
    o += "]}";
  }
  o += "]}";
  return Dup(o);
}

HOST_EXPORT void xla_amd_host_free(char* p) { free(p); }
