"""Text in, text out: a model folder with a tokenizer.json and a chat template of
its own (both made here with the `tokenizers` library, a word-level vocabulary of
the tiny model's size), through the encoding helpers, LLM.generate and the command
line.  The ids that reach the model are checked against the tokenizer's own, and
the generated ids against the plain implementation."""

import json
import shutil

import pytest

from .tiny import CONFIGS, make_model_dir

WORDS = ["<|user|>", "<|assistant|>", "<|end|>", "the", "sky", "is", "blue", "why", "tell", "me", "a", "story", "?", "."]
TEMPLATE = "{% for m in messages %}<|{{ m['role'] }}|> {{ m['content'] }} <|end|> {% endfor %}{% if add_generation_prompt %}<|assistant|>{% endif %}"


def add_tokenizer(folder):
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import WhitespaceSplit

    vocab = {w: i for i, w in enumerate(WORDS)}
    vocab["<unk>"] = len(WORDS)
    tok = Tokenizer(WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = WhitespaceSplit()
    tok.save(str(folder / "tokenizer.json"))
    (folder / "tokenizer_config.json").write_text(json.dumps({"chat_template": TEMPLATE}))
    return vocab


@pytest.fixture(scope="module")
def text_model(tmp_path_factory):
    root = tmp_path_factory.mktemp("text_models")
    src = make_model_dir("A", root, mode="unit")
    folder = root / "with_tokenizer"
    shutil.copytree(src, folder)
    return folder, add_tokenizer(folder)


def test_the_chat_template_and_the_encoding_are_the_folders_own(text_model):
    from shrike_amd.engine.llm_engine import _encode, _load_tokenizer, apply_chat_template

    folder, vocab = text_model
    text = apply_chat_template(folder, [{"role": "user", "content": "why is the sky blue ?"}])
    assert text == "<|user|> why is the sky blue ? <|end|> <|assistant|>"
    tok = _load_tokenizer(folder)
    plain_ids = _encode(tok, folder, "tell me a story .", chat=False)
    assert plain_ids == [vocab[w] for w in "tell me a story .".split()]
    chat_ids = _encode(tok, folder, "tell me a story .", chat=True)
    assert chat_ids == [vocab["<|user|>"], *plain_ids, vocab["<|end|>"], vocab["<|assistant|>"]]
    assert _encode(tok, folder, "tell me a fable", chat=False)[-1] == vocab["<unk>"]
    with pytest.raises(ValueError, match="tokenizer"):
        _encode(None, folder, "x", chat=False)


@pytest.mark.gpu
def test_text_prompts_through_generate_and_the_command_line(text_model, capsys):
    from shrike_amd import LLM, SamplingParams
    from shrike_amd.__main__ import main

    from .plain.model import PlainModel

    folder, vocab = text_model
    assert max(vocab.values()) < CONFIGS["A"]["vocab_size"]
    llm = LLM(str(folder), dtype="float32", block_size=4, num_kv_blocks=64)
    sampling = SamplingParams(max_new_tokens=6, ignore_eos=True)
    prompts = ["why is the sky blue ?", "tell me a story ."]
    from_text = llm.generate(prompts, sampling, chat=True)
    wrap = lambda ids: [vocab["<|user|>"], *ids, vocab["<|end|>"], vocab["<|assistant|>"]]  # noqa: E731
    ids = [wrap([vocab[w] for w in p.split()]) for p in prompts]
    assert from_text == llm.generate(ids, sampling, chat=False)
    plain = PlainModel(folder)
    for prompt_ids, new in zip(ids, from_text):
        seq = list(prompt_ids)
        for tok in new:
            assert tok == int(plain.logits(seq)[-1].argmax())
            seq.append(tok)
    # the command line prints the tokenizer's text for the generated ids
    rc = main(["--model", str(folder), "--dtype", "float32", "--max-tokens", "6", "--ignore-eos",
               "--block-size", "4", "--num-kv-blocks", "64", prompts[0]])
    assert rc in (0, None)
    # (piece by piece as the tokens arrive: a word-level tokenizer knows no spaces between pieces)
    printed = capsys.readouterr().out.replace(" ", "")
    assert llm.engine.tokenizer.decode(from_text[0], skip_special_tokens=True).replace(" ", "") in printed
