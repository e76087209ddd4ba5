"""Text in, text out on the GPU: the chat template, the tokenizer, a generation loop and the
streaming detokenizer driven the way the reference's session does it
(/root/reference/src/main.rs:651-741), on the tiny synthetic model with the fixture tokenizer
(its 1115 ids are within the model's 2048-row vocabulary). What is checked: the streamed
segments concatenate to the detokenizer's text; that text is the decode of the emitted tokens
(minus the generation's one leading space); the speculative loop streams the same text as the
plain one; an end-of-sequence id stops the generation and is not shown."""
import importlib
import os

import pytest

import synth

pytestmark = pytest.mark.gpu

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tokenizer")
MESSAGES = [{"role": "system", "content": "Be brief."}, {"role": "user", "content": "It's 9 o'clock; say hi to São Paulo"}]


def test_chat_generate_streams_text(orn, ctx):
    text = importlib.import_module("ornith-rs_amd.text")
    s = synth.SynthModel(synth.TINY, seed=11)
    ws = s.upload(orn, ctx)
    model = orn.TextModel(ctx, ws, s.text_config(orn))
    tk = text.Tokenizer(FIX)
    try:
        segs = []
        caches = model.make_cache(256, 4)
        out, fed = text.chat_generate(tk, MESSAGES, model, caches, 24, on_text=segs.append)
        caches.close()
        assert len(fed) == 24 or fed[-1] in tk.eos_ids
        shown = [t for t in fed if t not in tk.eos_ids]
        whole = tk.decode(shown)
        assert "".join(segs) == out
        if "\x00" not in whole:
            assert out == (whole[1:] if whole.startswith(" ") else whole)
        # the speculative loop emits the same tokens, so it streams the same text
        head = orn.MtpHead(model, ws, 64)
        caches = model.make_cache(256, 4)
        out2, fed2 = text.chat_generate(tk, MESSAGES, model, caches, 24, head=head, depth=2)
        caches.close()
        head.close()
        assert fed2 == fed and out2 == out
        # an end-of-sequence id stops the generation and is not shown: declare the third token one
        stop = fed[2]
        caches = model.make_cache(256, 4)
        out3, fed3 = text.chat_generate(tk, MESSAGES, model, caches, 24, eos_ids=tk.eos_ids + [stop])
        caches.close()
        first = fed.index(stop)
        assert fed3 == fed[:first + 1]
        whole3 = tk.decode(fed3[:-1])
        if "\x00" not in whole3:
            assert out3 == (whole3[1:] if whole3.startswith(" ") else whole3)
    finally:
        tk.close()
        model.close()
        ws.close()
