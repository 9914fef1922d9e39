"""The text front end of a model folder: tokenizer.json, BOS handling, chat template, stop ids and
sampling defaults (no GPU)."""
import json

import pytest

from gibbs_amd.text import open_text


def write_folder(path, template=None, generation=None, bos="<s>", write_config=True):
    from tokenizers import Tokenizer, models, pre_tokenizers
    vocab = {w: i for i, w in enumerate(["<unk>", "<s>", "</s>", "<|user|>", "<|assistant|>", "hello", "world", "how", "are", "you"])}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.add_special_tokens(["<s>", "</s>", "<|user|>", "<|assistant|>"])
    tok.save(str(path / "tokenizer.json"))
    cfg = {"eos_token": {"content": "</s>"}}
    if bos:
        cfg["bos_token"] = bos
    if template:
        cfg["chat_template"] = template
    (path / "tokenizer_config.json").write_text(json.dumps(cfg))
    if write_config:
        (path / "config.json").write_text(json.dumps({"eos_token_id": 2}))
    if generation:
        (path / "generation_config.json").write_text(json.dumps(generation))


TEMPLATE = ("{{ bos_token }}{% for m in messages %}<|{{ m['role'] }}|> {{ m['content'] }} {% endfor %}"
            "{% if add_generation_prompt %}<|assistant|>{% endif %}")


def test_encode_prepends_one_bos_and_decodes(tmp_path):
    write_folder(tmp_path)
    t = open_text(str(tmp_path))
    assert t.bos_id == 1 and t.chat_template is None
    assert t.encode("hello world") == [1, 5, 6]
    assert t.encode("<s> hello") == [1, 5], "a text that starts with BOS gets no second one"
    assert t.prompt_ids("how are you") == [1, 7, 8, 9]
    assert t.decode([5, 6]) == "hello world"
    assert set(t.stop_ids) == {2, 3, 4}, "the end id of config.json and the special tokens, but not BOS"
    assert t.sampling_defaults is None
    with pytest.raises(ValueError, match="no chat template"):
        t.apply_chat_template([("user", "hello")])
    assert open_text(str(tmp_path / "nowhere")) is None


def test_chat_template_and_sampling_defaults(tmp_path):
    write_folder(tmp_path, template=TEMPLATE, generation={"do_sample": False, "eos_token_id": [2, 9]})
    t = open_text(str(tmp_path))
    text = t.apply_chat_template([("user", "hello world")])
    assert text == "<s><|user|> hello world <|assistant|>"
    assert t.prompt_ids("hello world") == [1, 3, 5, 6, 4], "one BOS: the template wrote it"
    assert t.apply_chat_template([("user", "hello")], add_generation_prompt=False) == "<s><|user|> hello "
    assert t.sampling_defaults == (0.0, 1.0) and 9 in t.stop_ids
    write_folder(tmp_path, template="{{ raise_exception('no system role') }}", generation={"temperature": 0.3, "top_p": 0.8})
    t = open_text(str(tmp_path))
    assert t.sampling_defaults == (0.3, 0.8)
    with pytest.raises(Exception, match="no system role"):
        t.apply_chat_template([("user", "x")])
