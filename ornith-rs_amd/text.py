"""ctypes mirror of the library's text entry points (tokenizer, streaming detokenizer, chat
template): the reference's Tokenizer / Detokenizer / apply_chat_template
(/root/reference/src/tokenizer/mod.rs, src/chat.rs) for tests and tools. Host only.
"""
import ctypes as C
import json

from . import _check, lib

TOKENIZER_JSON, TRANSFORMERS = 0, 1


def _text_out(call, what):
    """Runs a (buffer, capacity, count) style call twice: size query, then the copy."""
    n = C.c_size_t()
    _check(call(None, 0, C.byref(n)), what)
    buf = C.create_string_buffer(max(n.value, 1))
    _check(call(buf, n.value, C.byref(n)), what)
    return buf.raw[:n.value]


class Tokenizer:
    def __init__(self, model_dir, dialect=TOKENIZER_JSON):
        h = C.c_void_p()
        _check(lib().ornith_tokenizer_load(str(model_dir).encode(), dialect, C.byref(h)), "tokenizer_load")
        self.h = h

    @property
    def vocab_size(self):
        n = C.c_size_t()
        _check(lib().ornith_tokenizer_vocab_size(self.h, C.byref(n)), "tokenizer_vocab_size")
        return n.value

    def encode(self, text):
        raw = text if isinstance(text, bytes) else text.encode("utf-8")
        n = C.c_size_t()
        _check(lib().ornith_tokenizer_encode(self.h, raw, C.c_size_t(len(raw)), None, 0, C.byref(n)), "tokenizer_encode")
        ids = (C.c_uint32 * max(n.value, 1))()
        _check(lib().ornith_tokenizer_encode(self.h, raw, C.c_size_t(len(raw)), ids, C.c_size_t(n.value), C.byref(n)),
               "tokenizer_encode")
        return list(ids[:n.value])

    def decode(self, ids):
        arr = (C.c_uint32 * max(len(ids), 1))(*ids)
        return _text_out(lambda b, c, n: lib().ornith_tokenizer_decode(self.h, arr, C.c_size_t(len(ids)), b, C.c_size_t(c), n),
                         "tokenizer_decode").decode("utf-8")

    def token(self, i):
        return _text_out(lambda b, c, n: lib().ornith_tokenizer_token(self.h, C.c_uint32(i), b, C.c_size_t(c), n),
                         "tokenizer_token").decode("utf-8")

    def id(self, token):
        out = C.c_uint32()
        rc = lib().ornith_tokenizer_id(self.h, token.encode("utf-8"), C.byref(out))
        return None if rc else out.value

    def is_special(self, i):
        return bool(lib().ornith_tokenizer_is_special(self.h, C.c_uint32(i)))

    @property
    def eos_ids(self):
        n = C.c_size_t()
        _check(lib().ornith_tokenizer_eos_ids(self.h, None, 0, C.byref(n)), "tokenizer_eos_ids")
        ids = (C.c_uint32 * max(n.value, 1))()
        _check(lib().ornith_tokenizer_eos_ids(self.h, ids, C.c_size_t(n.value), C.byref(n)), "tokenizer_eos_ids")
        return list(ids[:n.value])

    def detokenizer(self):
        return Detokenizer(self)

    def close(self):
        if self.h:
            lib().ornith_tokenizer_destroy(self.h)
            self.h = None


class Detokenizer:
    def __init__(self, tk):
        self.tk = tk  # keeps the tokenizer alive
        h = C.c_void_p()
        _check(lib().ornith_detokenizer_create(tk.h, C.byref(h)), "detokenizer_create")
        self.h = h

    def add_token(self, t):
        _check(lib().ornith_detokenizer_add_token(self.h, C.c_uint32(t)), "detokenizer_add_token")

    def finalize(self):
        _check(lib().ornith_detokenizer_finalize(self.h), "detokenizer_finalize")

    def last_segment(self):
        return _text_out(lambda b, c, n: lib().ornith_detokenizer_last_segment(self.h, b, C.c_size_t(c), n),
                         "detokenizer_last_segment").decode("utf-8")

    @property
    def text(self):
        return _text_out(lambda b, c, n: lib().ornith_detokenizer_text(self.h, b, C.c_size_t(c), n),
                         "detokenizer_text").decode("utf-8")

    def close(self):
        if self.h:
            lib().ornith_detokenizer_destroy(self.h)
            self.h = None


def split_pattern(dialect):
    f = lib().ornith_tokenizer_split_pattern
    f.restype = C.c_char_p
    return f(dialect).decode()


def nfc(text):
    raw = text.encode("utf-8")
    return _text_out(lambda b, c, n: lib().ornith_text_nfc(raw, C.c_size_t(len(raw)), b, C.c_size_t(c), n),
                     "text_nfc").decode("utf-8")


def pre_split(text, dialect=TOKENIZER_JSON):
    raw = text.encode("utf-8")
    n = C.c_size_t()
    _check(lib().ornith_text_pre_split(raw, C.c_size_t(len(raw)), dialect, None, 0, C.byref(n)), "text_pre_split")
    ends = (C.c_size_t * max(n.value, 1))()
    _check(lib().ornith_text_pre_split(raw, C.c_size_t(len(raw)), dialect, ends, C.c_size_t(n.value), C.byref(n)),
           "text_pre_split")
    out, a = [], 0
    for e in ends[:n.value]:
        out.append(raw[a:e].decode("utf-8"))
        a = e
    return out


def char_class(cp):
    return lib().ornith_text_char_class(C.c_uint32(cp))


def apply_chat_template(messages, tools=None, add_generation_prompt=True, enable_thinking=False):
    """messages / tools: Python lists as tokenizer.apply_chat_template takes them (or JSON text)."""
    m = messages if isinstance(messages, (str, bytes)) else json.dumps(messages, ensure_ascii=False)
    m = m.encode("utf-8") if isinstance(m, str) else m
    t = None
    if tools:
        t = tools if isinstance(tools, (str, bytes)) else json.dumps(tools, ensure_ascii=False)
        t = t.encode("utf-8") if isinstance(t, str) else t
    return _text_out(lambda b, c, n: lib().ornith_chat_apply_template(
        m, C.c_size_t(len(m)), t, C.c_size_t(len(t) if t else 0), int(add_generation_prompt), int(enable_thinking),
        b, C.c_size_t(c), n), "chat_apply_template").decode("utf-8")


def json_dumps(text):
    raw = text.encode("utf-8") if isinstance(text, str) else text
    return _text_out(lambda b, c, n: lib().ornith_json_dumps(raw, C.c_size_t(len(raw)), b, C.c_size_t(c), n),
                     "json_dumps").decode("utf-8")


def chat_generate(tk, messages, model, caches, max_tokens, head=None, frspec=None, depth=1, sampler=None,
                  tools=None, enable_thinking=False, prefill_step=2048, on_text=None, eos_ids=None):
    """Text in, text out, the way the reference's session drives the loops
    (/root/reference/src/main.rs:651-741): render the chat template, encode, generate with an
    emit callback that stops at an end-of-sequence id, streams every other token through the
    detokenizer and stops after max_tokens. eos_ids overrides the tokenizer's own stop ids.
    Returns (text, emitted token ids incl. the stop)."""
    from . import engine
    prompt = tk.encode(apply_chat_template(messages, tools, True, enable_thinking))
    detok, eos, fed, n = tk.detokenizer(), set(tk.eos_ids if eos_ids is None else eos_ids), [], [0]

    def emit(t):
        fed.append(t)
        if t in eos:
            return False
        detok.add_token(t)
        n[0] += 1
        seg = detok.last_segment()
        if seg and on_text:
            on_text(seg)
        return n[0] < max_tokens

    if head is not None:
        engine.generate_step_mtp(model, head, frspec, caches, prompt, depth, max_tokens, sampler, prefill_step, on_token=emit)
    else:
        engine.generate_step(model, caches, prompt, max_tokens, sampler, prefill_step, on_token=emit)
    detok.finalize()
    seg = detok.last_segment()
    if seg and on_text:
        on_text(seg)
    out = detok.text
    detok.close()
    return out, fed
