// The model's chat template, written out as code, and the JSON writer its tool blocks need
// (host only).
//
//   apply_chat_template, Message, Content, ToolCall, TemplateError   /root/reference/src/chat.rs:1-352
//   Value::to_json (json.dumps(v, ensure_ascii=False))               /root/reference/src/json.rs
//
// The template, in order: a system block (the tool list with its calling convention when tools
// are given, then the system message's own text; else the first message if it is a system
// one); a backwards scan that only ever raises "No user query found"; the messages by role;
// the generation prompt with an open or an already-closed <think> block. Every content goes
// through |trim, which is Python's str.strip().
//
// Messages cross the C boundary as the JSON a caller of tokenizer.apply_chat_template would
// pass: [{"role", "content": string | [parts] | null, "reasoning_content", "tool_calls"}].
#include <cmath>

#include "json.h"
#include "rt.h"
#include "text.h"

using namespace orn_json;

namespace {

// ---- json.dumps(v, ensure_ascii=False) ---------------------------------------------
void dump_string(const std::string& s, std::string& out) {
  out.push_back('"');
  for (unsigned char c : s) {
    switch (c) {
      case '"': out += "\\\""; break;
      case '\\': out += "\\\\"; break;
      case '\n': out += "\\n"; break;
      case '\r': out += "\\r"; break;
      case '\t': out += "\\t"; break;
      case '\b': out += "\\b"; break;
      case '\f': out += "\\f"; break;
      default:
        if (c < 0x20) {
          char buf[8];
          snprintf(buf, sizeof buf, "\\u%04x", c);
          out += buf;
        } else {
          out.push_back((char)c);  // non-ASCII stays as it is
        }
    }
  }
  out.push_back('"');
}

// Python's repr(float): the shortest digits that read back to the same double; exponent form
// below 1e-4 and from 1e16 up; a whole number keeps its ".0"
void dump_float(double v, std::string& out) {
  if (std::isnan(v)) { out += "NaN"; return; }
  if (std::isinf(v)) { out += v > 0 ? "Infinity" : "-Infinity"; return; }
  char buf[40];
  int prec = 1;
  for (; prec <= 17; ++prec) {
    snprintf(buf, sizeof buf, "%.*e", prec - 1, v);
    if (strtod(buf, nullptr) == v) break;
  }
  // buf = d.ddddde[+-]XX
  std::string digits;
  bool neg = false;
  const char* p = buf;
  if (*p == '-') { neg = true; ++p; }
  for (; *p && *p != 'e'; ++p)
    if (*p != '.') digits.push_back(*p);
  const int exp10 = atoi(p + 1);
  while (digits.size() > 1 && digits.back() == '0') digits.pop_back();
  std::string r = neg ? "-" : "";
  if (exp10 < -4 || exp10 >= 16) {
    r += digits.substr(0, 1);
    if (digits.size() > 1) r += "." + digits.substr(1);
    char e[16];
    snprintf(e, sizeof e, "e%c%02d", exp10 < 0 ? '-' : '+', exp10 < 0 ? -exp10 : exp10);
    r += e;
  } else if (exp10 < 0) {
    r += "0." + std::string((size_t)(-exp10 - 1), '0') + digits;
  } else if ((int)digits.size() <= exp10 + 1) {
    r += digits + std::string((size_t)(exp10 + 1 - (int)digits.size()), '0') + ".0";
  } else {
    r += digits.substr(0, (size_t)exp10 + 1) + "." + digits.substr((size_t)exp10 + 1);
  }
  out += r;
}

void dump(const JVal& v, std::string& out) {
  switch (v.kind) {
    case JVal::Null: out += "null"; break;
    case JVal::Bool: out += v.b ? "true" : "false"; break;
    case JVal::Str: dump_string(v.str, out); break;
    case JVal::Num:
      if (v.is_int) out += v.raw == "-0" ? "0" : v.raw;  // an int literal reads as a Python int
      else dump_float(v.num, out);
      break;
    case JVal::Arr:
      out.push_back('[');
      for (size_t i = 0; i < v.arr.size(); ++i) {
        if (i) out += ", ";
        dump(v.arr[i], out);
      }
      out.push_back(']');
      break;
    case JVal::Obj:
      out.push_back('{');
      for (size_t i = 0; i < v.obj.size(); ++i) {
        if (i) out += ", ";
        dump_string(v.obj[i].first, out);
        out += ": ";
        dump(v.obj[i].second, out);
      }
      out.push_back('}');
      break;
  }
}

// Python's str.strip(): str.isspace() characters off both ends
std::string py_strip(const std::string& s) {
  std::vector<uint32_t> cps;
  if (!orn_text::utf8_decode(s.data(), s.size(), &cps)) return s;
  size_t a = 0, b = cps.size();
  while (a < b && orn_text::is_py_space(cps[a])) ++a;
  while (b > a && orn_text::is_py_space(cps[b - 1])) --b;
  std::string out;
  for (size_t i = a; i < b; ++i) orn_text::utf8_append(out, cps[i]);
  return out;
}

bool starts_with(const std::string& s, const char* p) { return s.compare(0, strlen(p), p) == 0; }
bool ends_with(const std::string& s, const char* p) {
  const size_t n = strlen(p);
  return s.size() >= n && s.compare(s.size() - n, n, p) == 0;
}
std::string rstrip_nl(std::string s) {
  while (!s.empty() && s.back() == '\n') s.pop_back();
  return s;
}
std::string lstrip_nl(const std::string& s) {
  size_t i = 0;
  while (i < s.size() && s[i] == '\n') ++i;
  return s.substr(i);
}

const char* kToolCallInstructions =
    "\n\nIf you choose to call a function ONLY reply in the following format with NO suffix:\n\n"
    "<tool_call>\n<function=example_function_name>\n<parameter=example_parameter_1>\nvalue_1\n</parameter>\n"
    "<parameter=example_parameter_2>\nThis is the value for the second parameter\nthat can span\nmultiple lines\n"
    "</parameter>\n</function>\n</tool_call>\n\n<IMPORTANT>\nReminder:\n"
    "- Function calls MUST follow the specified format: an inner <function=...></function> block must be nested "
    "within <tool_call></tool_call> XML tags\n"
    "- Required parameters MUST be specified\n"
    "- You may provide optional reasoning for your function call in natural language BEFORE the function call, "
    "but NOT after\n"
    "- If there is no function call available, answer the question like normal with your current knowledge and do "
    "not tell the user about function calls\n</IMPORTANT>";

enum Role { SYSTEM, USER, ASSISTANT, TOOL };

int role_of(const JVal& m, Role* out) {
  const JVal* r = m.get("role");
  ORN_REQUIRE(r && r->kind == JVal::Str, "chat_template: a message has no role");
  if (r->str == "system") *out = SYSTEM;
  else if (r->str == "user") *out = USER;
  else if (r->str == "assistant") *out = ASSISTANT;
  else if (r->str == "tool") *out = TOOL;
  else return ornith_fail(ORNITH_ERR_INVALID, "chat_template: unknown role \"%s\"", r->str.c_str());
  return ORNITH_OK;
}

// render_content(...) | trim: a string as it is; a list of parts with an image / video
// placeholder per visual item (not allowed in a system message) and the text items' text;
// null or absent as empty
int rendered(const JVal& m, bool is_system, std::string* out) {
  std::string s;
  const JVal* c = m.get("content");
  if (c && c->kind == JVal::Str) {
    s = c->str;
  } else if (c && c->kind == JVal::Arr) {
    for (auto& p : c->arr) {
      const JVal* ty = p.get("type");
      const bool image = p.get("image") || p.get("image_url") || (ty && ty->kind == JVal::Str && ty->str == "image");
      const bool video = p.get("video") || (ty && ty->kind == JVal::Str && ty->str == "video");
      const JVal* text = p.get("text");
      if (image) {
        if (is_system) return ornith_fail(ORNITH_ERR_INVALID, "System message cannot contain images.");
        s += "<|vision_start|><|image_pad|><|vision_end|>";
      } else if (video) {
        if (is_system) return ornith_fail(ORNITH_ERR_INVALID, "System message cannot contain videos.");
        s += "<|vision_start|><|video_pad|><|vision_end|>";
      } else if (text && text->kind == JVal::Str) {
        s += text->str;
      } else {
        return ornith_fail(ORNITH_ERR_INVALID, "chat_template: unexpected item type in content");
      }
    }
  } else if (c && c->kind != JVal::Null) {
    return ornith_fail(ORNITH_ERR_INVALID, "chat_template: content is neither a string, a list nor null");
  }
  *out = py_strip(s);
  return ORNITH_OK;
}

int apply(const JVal& messages, const JVal* tools, bool add_generation_prompt, bool enable_thinking, std::string* res) {
  ORN_REQUIRE(messages.kind == JVal::Arr, "chat_template: messages is not a list");
  if (messages.arr.empty()) return ornith_fail(ORNITH_ERR_INVALID, "No messages provided.");
  const size_t n = messages.arr.size();
  std::vector<Role> roles(n);
  for (size_t i = 0; i < n; ++i)
    if (int rc = role_of(messages.arr[i], &roles[i])) return rc;
  std::string out;
  const bool have_tools = tools && tools->kind == JVal::Arr && !tools->arr.empty();
  if (have_tools) {
    out += "<|im_start|>system\n# Tools\n\nYou have access to the following functions:\n\n<tools>";
    for (auto& t : tools->arr) {
      out.push_back('\n');
      dump(t, out);
    }
    out += "\n</tools>";
    out += kToolCallInstructions;
    if (roles[0] == SYSTEM) {
      std::string content;
      if (int rc = rendered(messages.arr[0], true, &content)) return rc;
      if (!content.empty()) out += "\n\n" + content;  // an empty system message adds nothing here
    }
    out += "<|im_end|>\n";
  } else if (roles[0] == SYSTEM) {
    std::string content;
    if (int rc = rendered(messages.arr[0], true, &content)) return rc;
    out += "<|im_start|>system\n" + content + "<|im_end|>\n";
  }

  // the backwards scan: its index is never read, its "no real user query" error is
  bool multi_step_tool = true;
  for (size_t k = n; k-- > 0;) {
    if (multi_step_tool && roles[k] == USER) {
      std::string content;
      if (int rc = rendered(messages.arr[k], false, &content)) return rc;
      if (!(starts_with(content, "<tool_response>") && ends_with(content, "</tool_response>"))) multi_step_tool = false;
    }
  }
  if (multi_step_tool) return ornith_fail(ORNITH_ERR_INVALID, "No user query found in messages.");

  for (size_t i = 0; i < n; ++i) {
    const JVal& m = messages.arr[i];
    std::string content;
    if (int rc = rendered(m, false, &content)) return rc;
    switch (roles[i]) {
      case SYSTEM:
        if (i != 0) return ornith_fail(ORNITH_ERR_INVALID, "System message must be at the beginning.");
        break;  // already emitted above
      case USER:
        out += "<|im_start|>user\n" + content + "<|im_end|>\n";
        break;
      case ASSISTANT: {
        std::string reasoning;
        const JVal* rc_ = m.get("reasoning_content");
        if (rc_ && rc_->kind == JVal::Str) {
          reasoning = rc_->str;
        } else if (content.find("</think>") != std::string::npos) {
          // reasoning: what stands between the last <think> before the first </think> and
          // that </think>; content: what follows the last </think>
          const std::string head = rstrip_nl(content.substr(0, content.find("</think>")));
          const size_t open = head.rfind("<think>");
          reasoning = lstrip_nl(open == std::string::npos ? head : head.substr(open + 7));
          content = lstrip_nl(content.substr(content.rfind("</think>") + 8));
        }
        out += "<|im_start|>assistant\n<think>\n" + py_strip(reasoning) + "\n</think>\n\n" + content;
        const JVal* calls = m.get("tool_calls");
        if (calls && calls->kind == JVal::Arr) {
          for (size_t j = 0; j < calls->arr.size(); ++j) {
            const JVal* call = &calls->arr[j];
            if (const JVal* f = call->get("function")) call = f;  // the wrapped shape
            const JVal* name = call->get("name");
            ORN_REQUIRE(name && name->kind == JVal::Str, "chat_template: a tool call has no name");
            if (j > 0) out.push_back('\n');
            else if (!py_strip(content).empty()) out += "\n\n";
            out += "<tool_call>\n<function=" + name->str + ">\n";
            const JVal* args = call->get("arguments");
            if (args && args->kind == JVal::Obj)
              for (auto& kv : args->obj) {
                out += "<parameter=" + kv.first + ">\n";
                if (kv.second.kind == JVal::Str) out += kv.second.str;  // a string goes in raw
                else dump(kv.second, out);
                out += "\n</parameter>\n";
              }
            out += "</function>\n</tool_call>";
          }
        }
        out += "<|im_end|>\n";
        break;
      }
      case TOOL:
        // a leading tool message opens no user block (the template has no previous item there)
        if (i > 0 && roles[i - 1] != TOOL) out += "<|im_start|>user";
        out += "\n<tool_response>\n" + content + "\n</tool_response>";
        if (i + 1 == n || roles[i + 1] != TOOL) out += "<|im_end|>\n";
        break;
    }
  }
  if (add_generation_prompt) out += enable_thinking ? "<|im_start|>assistant\n<think>\n" : "<|im_start|>assistant\n<think>\n\n</think>\n\n";
  *res = out;
  return ORNITH_OK;
}

int copy_out(const std::string& s, char* out, size_t cap, size_t* n_out, const char* who) {
  if (n_out) *n_out = s.size();
  if (!out) return ORNITH_OK;
  ORN_REQUIRE(cap >= s.size(), "%s: %zu bytes do not fit the buffer (%zu)", who, s.size(), cap);
  memcpy(out, s.data(), s.size());
  return ORNITH_OK;
}

}  // namespace

extern "C" {

int ornith_chat_apply_template(const char* messages_json, size_t messages_len, const char* tools_json,
                               size_t tools_len, int add_generation_prompt, int enable_thinking, char* out,
                               size_t cap, size_t* n_out) {
  ORN_REQUIRE(messages_json, "chat_apply_template: null argument");
  JVal messages, tools;
  std::string err;
  ORN_REQUIRE(json_parse(messages_json, messages_len, &messages, &err), "chat_apply_template: messages: %s", err.c_str());
  if (tools_json && tools_len)
    ORN_REQUIRE(json_parse(tools_json, tools_len, &tools, &err), "chat_apply_template: tools: %s", err.c_str());
  std::string res;
  if (int rc = apply(messages, tools_json && tools_len ? &tools : nullptr, add_generation_prompt != 0,
                     enable_thinking != 0, &res))
    return rc;
  return copy_out(res, out, cap, n_out, "chat_apply_template");
}

int ornith_json_dumps(const char* json, size_t len, char* out, size_t cap, size_t* n_out) {
  ORN_REQUIRE(json, "json_dumps: null argument");
  JVal v;
  std::string err;
  ORN_REQUIRE(json_parse(json, len, &v, &err), "json_dumps: %s", err.c_str());
  std::string s;
  dump(v, s);
  return copy_out(s, out, cap, n_out, "json_dumps");
}

}  // extern "C"
