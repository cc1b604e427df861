"""Text in and out through a tokenizer in the model folder (reference: kvcore/utils/
tokenizer.py:15-114).  The tokenizer here is a word-level toy made on the spot."""

from __future__ import annotations

import json

import pytest

from kvcore_amd.engine.tokenizer import TokenizerManager


def make_tokenizer_folder(folder):
    from tokenizers import Tokenizer, models, pre_tokenizers

    words = ["<unk>", "<eos>", "<|user|>", "<|assistant|>", "<|system|>", "hello", "world", "how", "are", "you", "fine"]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    folder.mkdir(parents=True, exist_ok=True)
    tok.save(str(folder / "tokenizer.json"))
    template = ("{% for m in messages %}<|{{ m['role'] }}|> {{ m['content'] }} {% endfor %}"
                "{% if add_generation_prompt %}<|assistant|>{% endif %}")
    (folder / "tokenizer_config.json").write_text(json.dumps({
        "tokenizer_class": "PreTrainedTokenizerFast", "eos_token": "<eos>", "unk_token": "<unk>",
        "chat_template": template}))
    return words


def test_no_tokenizer_files_means_no_tokenizer(tmp_path):
    assert TokenizerManager.from_model_source(tmp_path) is None


def test_chat_template_decode_and_stop_ids(tmp_path):
    words = make_tokenizer_folder(tmp_path / "m")
    manager = TokenizerManager.from_model_source(tmp_path / "m")
    assert manager is not None
    ids = manager.encode_messages([{"role": "system", "content": "hello"},
                                   {"role": "user", "content": "how are you"}])
    # the template's text, word by word, with the generation prompt at the end
    assert [words[i] for i in ids] == ["<|system|>", "hello", "<|user|>", "how", "are", "you", "<|assistant|>"]
    assert manager.decode([words.index("fine"), words.index("world"), words.index("<eos>")]) == "fine world"
    assert manager.get_stop_token_ids() == {words.index("<eos>")}
    with pytest.raises(ValueError):
        manager.encode_messages([{"role": "robot", "content": "hello"}])
    with pytest.raises(ValueError):
        manager.encode_messages([{"role": "user", "content": 5}])
