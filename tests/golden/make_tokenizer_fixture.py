"""Writes tests/golden/tokenizer/: a small byte-level BPE tokenizer of the model's pipeline shape
and what the `tokenizers` library (the implementation the reference tests itself against,
/root/reference/tests/tokenizer.rs:1-8, tools/dump_tokenizer.py) makes of a set of strings.

    python tests/golden/make_tokenizer_fixture.py

The real artifact's tokenizer.json is not available offline, so the vocabulary is trained here
(seeded, a few hundred merges over a synthetic multilingual corpus); the pipeline around it is
the model's: NFC -> Split(the pattern, Isolated) + ByteLevel -> BPE, added tokens split off the
raw text first. Nothing of the reference is imported or run. Written:

  tokenizer.json, tokenizer_config.json, generation_config.json   the files Tokenizer::load reads
  cases.json     strings, their ids under both split patterns, decode(ids), NFC outputs, the
                 pre-tokenizer's pieces, the token string of every id
  classes.json   the code points oniguruma puts in \\p{L}, \\p{M}, \\p{N} and \\s, as ranges, read
                 back out of live Split pre-tokenizers
"""
import json
import os
import random

from tokenizers import AddedToken, Regex, Tokenizer, decoders, models, normalizers, pre_tokenizers, processors, trainers

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "tokenizer")

PATTERN_JSON = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?[\p{L}\p{M}]+|\p{N}| ?[^\s\p{L}\p{M}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
PATTERN_TRANSFORMERS = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"

PHRASES = [
    "The quick brown fox jumps over the lazy dog.", "It's 9 o'clock; they've gone, haven't they?", "I'LL BE BACK, SAID HE'D.",
    "Prices rose 12.5% to $1,234.56 in 2024.", "def f(x):\n    return x ** 2  # square\n", "a = [1, 2, 3]\n\n\nprint(a)\t\tdone",
    "Größe, façade, naïve, coöperate, São Paulo, Ångström", "Ελληνικά γράμματα και αριθμοί ١٢٣", "Привет, мир! Как дела?",
    "हिन्दी में लिखना क़ानून", "العَرَبِيَّة لغةٌ جميلة", "日本語のテキストと漢字、カタカナ", "한국어 텍스트 각 갂", "emoji ☺️ 👍🏽 ✈️ done",
    "é ä ộ Ḑ̇ decomposed", "각 jamo", "tabs\tand  double  spaces   and nbsp　ideographic",
    "line one\r\nline two\rline three\n\n  indented", "snake_case camelCase kebab-case 3.14159 0x1F", "<tag attr=\"v\">text</tag> && || != ==",
    "ǅ ǆ ﬁ ﬂ ſ long s's", "½ ² ③ Ⅷ ๔ numbers", "​ zero width   line sep \u0085 nel", "...!!!???---___***",
]

ADDED = [("<|endoftext|>", True), ("<|im_start|>", True), ("<|im_end|>", True), ("<|vision_start|>", True),
         ("<|vision_end|>", True), ("<|image_pad|>", True), ("<|video_pad|>", True), ("<think>", False), ("</think>", False),
         ("<tool_call>", False), ("</tool_call>", False), ("<|im_start|>x", False)]
CONFIG_ONLY = [("<|audio_start|>", True), ("<tts_pad>", True)]

CASES = PHRASES + [
    "", " ", "  ", "\n", " \n ", "a", " a", "a ", "don't", "it'ss", "it'ſs", "IT'S'T'RE'VE'M'LL'D", "'", "''s", "123abc", "--x",
    "  \n\n  x", "a   ", "a  b", "a  x", "a   b", "x\r\n\r\ny", "   \t\n", "a.\n\nb", "a !\r\n", " ?!", "  ?!",
    "हिन", "́abc", "á́́", "Å Ω Å", "क़ क़", "̈́", "ཷ",
    "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n", "<|im_start|>x<|im_start|>", "<|im_start", "<think></think><tool_call>",
    "<|audio_start|><tts_pad>", "a<|endoftext|>b<|endoftext|>", "é<|im_end|>é", "\U0001F468‍\U0001F469‍\U0001F467", "각", "가",
    "mixed: abc123def 4five6 ７８９ ٣٤", "tab\tsep\t\tcol", "UPPER lower MiXeD", "aaaaaaaaaaaaaaaa", "abababababab", "  leading and trailing  ",
]


def build(pattern, model=None):
    tok = Tokenizer(model if model is not None else models.BPE())
    tok.normalizer = normalizers.NFC()
    tok.pre_tokenizer = pre_tokenizers.Sequence([
        pre_tokenizers.Split(Regex(pattern), behavior="isolated", invert=False),
        pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    tok.decoder = decoders.ByteLevel()
    tok.post_processor = processors.ByteLevel(trim_offsets=False)
    return tok


def class_ranges(regex):
    """Code points a one-character oniguruma class matches, via a live Split pre-tokenizer."""
    pt = pre_tokenizers.Split(Regex(regex), behavior="removed")
    hit = []
    step = 0x4000
    cps = [c for c in range(0x110000) if not 0xD800 <= c <= 0xDFFF]
    for a in range(0, len(cps), step):
        chunk = cps[a:a + step]
        text = "".join(chr(c) for c in chunk)
        kept = set()
        for _, (s, e) in pt.pre_tokenize_str(text):
            kept.update(range(s, e))
        hit += [c for i, c in enumerate(chunk) if i not in kept]
    out = []
    for c in hit:
        if out and out[-1][1] + 1 == c:
            out[-1][1] = c
        else:
            out.append([c, c])
    return out


def main():
    os.makedirs(OUT, exist_ok=True)
    rng = random.Random(20260)
    corpus = []
    for _ in range(4000):
        k = rng.randint(1, 3)
        corpus.append(rng.choice(["", " ", "\n"]).join(rng.choice(PHRASES) for _ in range(k)))
    tok = build(PATTERN_JSON)
    trainer = trainers.BpeTrainer(vocab_size=1400, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), special_tokens=[],
                                  show_progress=False)
    tok.train_from_iterator(corpus, trainer)
    tok.add_tokens([AddedToken(c, special=s, normalized=False) for c, s in ADDED if not s])
    tok.add_special_tokens([AddedToken(c, special=True, normalized=False) for c, s in ADDED if s])
    tok.save(os.path.join(OUT, "tokenizer.json"))

    # the ids of the tokens only tokenizer_config.json knows follow the last one of tokenizer.json
    tj = json.load(open(os.path.join(OUT, "tokenizer.json")))
    next_id = max(t["id"] for t in tj["added_tokens"]) + 1
    dec = {}
    for t in tj["added_tokens"][:2]:      # the config repeats some of tokenizer.json's, as the artifact's does
        dec[str(t["id"])] = {k: t[k] for k in ("content", "lstrip", "normalized", "rstrip", "single_word", "special")}
    extra = []
    for c, s in CONFIG_ONLY:
        dec[str(next_id)] = dict(content=c, lstrip=False, normalized=False, rstrip=False, single_word=False, special=s)
        extra.append(AddedToken(c, special=s, normalized=False))
        next_id += 1
    json.dump(dict(add_bos_token=False, added_tokens_decoder=dec, eos_token="<|im_end|>", tokenizer_class="Qwen2Tokenizer"),
              open(os.path.join(OUT, "tokenizer_config.json"), "w"), indent=1)
    eos = [tok.token_to_id("<|im_end|>"), tok.token_to_id("<|endoftext|>")]
    json.dump(dict(eos_token_id=eos), open(os.path.join(OUT, "generation_config.json"), "w"))

    # the reference tokenizers: tokenizer.json + the config-only tokens, under each pattern
    full = Tokenizer.from_file(os.path.join(OUT, "tokenizer.json"))
    full.add_special_tokens(extra)
    other = Tokenizer.from_str(full.to_str())
    other.pre_tokenizer = build(PATTERN_TRANSFORMERS).pre_tokenizer
    nfc = normalizers.NFC()
    split_json = pre_tokenizers.Split(Regex(PATTERN_JSON), behavior="isolated")
    split_tr = pre_tokenizers.Split(Regex(PATTERN_TRANSFORMERS), behavior="isolated")
    cases = dict(
        text=CASES,
        ids_json=[full.encode(t, add_special_tokens=False).ids for t in CASES],
        ids_transformers=[other.encode(t, add_special_tokens=False).ids for t in CASES],
        nfc=[nfc.normalize_str(t) for t in CASES],
        pieces_json=[[p for p, _ in split_json.pre_tokenize_str(nfc.normalize_str(t))] for t in CASES],
        pieces_transformers=[[p for p, _ in split_tr.pre_tokenize_str(nfc.normalize_str(t))] for t in CASES],
        tokenmap=[full.id_to_token(i) for i in range(full.get_vocab_size(with_added_tokens=True))],
        pattern_json=PATTERN_JSON, pattern_transformers=PATTERN_TRANSFORMERS,
    )
    cases["decoded"] = [full.decode(ids, skip_special_tokens=False) for ids in cases["ids_json"]]
    # ids that split a multi-byte character over tokens: what decode makes of every prefix
    cases["prefix_decoded"] = [[full.decode(ids[:k], skip_special_tokens=False) for k in range(len(ids) + 1)]
                               for ids in cases["ids_json"][:40]]
    json.dump(cases, open(os.path.join(OUT, "cases.json"), "w"), ensure_ascii=True)
    json.dump({"L": class_ranges(r"\p{L}"), "M": class_ranges(r"\p{M}"), "N": class_ranges(r"\p{N}"),
               "s": class_ranges(r"\s")}, open(os.path.join(OUT, "classes.json"), "w"))
    print("vocab", full.get_vocab_size(with_added_tokens=True), "cases", len(CASES))


if __name__ == "__main__":
    main()
