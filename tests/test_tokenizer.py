"""The optional tokenizer of a model folder: loading, streaming detokenizer, chat template, prompt of the command line."""

import json
import os

import pytest

CORPUS = [
    "the quick brown fox jumps over the lazy dog",
    "pages of keys and values, a table of blocks for each request",
    "zwölf Boxkämpfer jagen Viktor quer über den großen Sylter Deich",
    "line one\nline two\n\nline four",
] * 4

TEMPLATE = (
    "{% for m in messages %}"
    "{% if m['role'] == 'tool' %}{{ raise_exception('no tools here') }}{% endif %}"
    "{{ bos_token }}<{{ m['role'] }}>{{ m['content'] }}{{ eos_token }}\n"
    "{% endfor %}"
    "{% if add_generation_prompt %}<assistant>{% if terse %}(short) {% endif %}{% endif %}"
)


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    """A byte-level BPE tokenizer trained here on a few lines, with so few merges that letters
    beyond ASCII take two tokens."""
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers, trainers

    d = tmp_path_factory.mktemp("tok")
    tok = Tokenizer(models.BPE())
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=300, special_tokens=["<|endoftext|>", "<|start|>"],
                                  initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), show_progress=False)
    tok.train_from_iterator([c for c in CORPUS if "ö" not in c], trainer)
    tok.save(os.path.join(d, "tokenizer.json"))
    with open(os.path.join(d, "tokenizer_config.json"), "w") as fh:
        json.dump({"bos_token": {"content": "<|start|>"}, "eos_token": "<|endoftext|>",
                   "chat_template": TEMPLATE}, fh)
    return str(d)


def test_folder_without_tokenizer_gives_none(tmp_path):
    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    assert load_tokenizer(str(tmp_path)) is None


def test_encode_decode_and_end_tokens(folder):
    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    tok = load_tokenizer(folder)
    for text in CORPUS[:4]:
        assert tok.decode(tok.encode(text)) == text
    assert tok.bos_token == "<|start|>" and tok.eos_token == "<|endoftext|>"
    assert tok.eos_token_ids == {0}  # from tokenizer_config.json, the config gave none
    assert load_tokenizer(folder, eos_token_ids=[7, 9]).eos_token_ids == {7, 9}  # the config's win
    assert load_tokenizer(folder, eos_token_ids=5).eos_token_ids == {5}
    tok.add_eos_token("<|start|>")
    tok.add_eos_token("17")
    assert tok.eos_token_ids == {0, 1, 17}
    with pytest.raises(ValueError, match="not a token"):
        tok.add_eos_token("no such token")


def test_streaming_detokenizer_equals_decoding_at_once(folder):
    """Segments add up to the whole text whatever the cuts; a letter whose bytes lie in two tokens
    appears only when it is complete."""
    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    tok = load_tokenizer(folder)
    for text in CORPUS[:4]:
        ids = tok.encode(text)
        if "ö" in text:
            assert len(ids) > len(text.encode()) // 3  # the split letters are really there
        det = tok.detokenizer
        pieces = []
        for t in ids:
            det.add_token(t)
            seg = det.last_segment
            assert "�" not in seg
            pieces.append(seg)
        det.finalize()
        pieces.append(det.last_segment)
        assert "".join(pieces) == text == det.text
        assert det.tokens == ids
        det.reset()
        assert det.text == "" and det.tokens == []


def test_chat_template(folder):
    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    tok = load_tokenizer(folder)
    assert tok.has_chat_template
    messages = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "the lazy dog"}]
    text = tok.apply_chat_template(messages, tokenize=False, add_generation_prompt=True)
    assert text == ("<|start|><system>be brief<|endoftext|>\n<|start|><user>the lazy dog<|endoftext|>\n<assistant>")
    assert tok.apply_chat_template(messages, tokenize=False, add_generation_prompt=True, terse=True).endswith(
        "<assistant>(short) ")
    ids = tok.apply_chat_template(messages, add_generation_prompt=True)
    assert ids == tok.encode(text, add_special_tokens=False) and ids[0] == 1 and 0 in ids
    going_on = messages + [{"role": "assistant", "content": "the quick "}]
    text = tok.apply_chat_template(going_on, tokenize=False, continue_final_message=True)
    assert text.endswith("<assistant>the quick")
    with pytest.raises(ValueError, match="no tools"):
        tok.apply_chat_template([{"role": "tool", "content": "x"}], tokenize=False)
    with pytest.raises(ValueError, match="exclude"):
        tok.apply_chat_template(going_on, add_generation_prompt=True, continue_final_message=True)


def test_a_template_file_wins_and_none_means_none(folder, tmp_path):
    import shutil

    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    shutil.copy(os.path.join(folder, "tokenizer.json"), tmp_path)
    tok = load_tokenizer(str(tmp_path))
    assert not tok.has_chat_template and tok.eos_token_ids == set()
    with pytest.raises(ValueError, match="no chat template"):
        tok.apply_chat_template([{"role": "user", "content": "x"}])
    shutil.copy(os.path.join(folder, "tokenizer_config.json"), tmp_path)
    with open(os.path.join(tmp_path, "chat_template.jinja"), "w") as fh:
        fh.write("{{ messages[-1]['content'] }}!")
    tok = load_tokenizer(str(tmp_path))
    assert tok.apply_chat_template([{"role": "user", "content": "fox"}], tokenize=False) == "fox!"


def test_the_command_lines_prompt(folder):
    """``--system-prompt``, ``--prefill-response``, ``--chat-template-config`` and ``--ignore-chat-template``."""
    from mlx_lm_amd.generate import IdTokenizer, chat_prompt, setup_arg_parser
    from mlx_lm_amd.tokenizer_utils import load_tokenizer

    tok = load_tokenizer(folder)
    parse = setup_arg_parser().parse_args
    args = parse(["--model", "x", "--system-prompt", "be brief"])
    ids = chat_prompt(tok, "the lazy dog", args)
    assert tok.decode(ids) == "<|start|><system>be brief<|endoftext|>\n<|start|><user>the lazy dog<|endoftext|>\n<assistant>"
    args = parse(["--model", "x", "--prefill-response", "the quick", "--chat-template-config", '{"terse": true}'])
    assert tok.decode(chat_prompt(tok, "fox", args)).endswith("<assistant>the quick")
    args = parse(["--model", "x", "--chat-template-config", '{"terse": true}'])
    assert tok.decode(chat_prompt(tok, "fox", args)).endswith("<assistant>(short) ")
    args = parse(["--model", "x", "--ignore-chat-template"])
    assert chat_prompt(tok, "fox", args) == "fox"
    assert chat_prompt(IdTokenizer(), "1 2 3", parse(["--model", "x"])) == "1 2 3"


def test_the_detokenizer_of_a_byte_level_vocabulary_looks_bytes_up(folder, tmp_path):
    """A byte-level vocabulary's tokens are fixed runs of bytes (the table covers all 256); any
    other vocabulary is decoded again from the last line break."""
    from tokenizers import Tokenizer, models, pre_tokenizers, trainers

    from mlx_lm_amd.tokenizer_utils import TokenizerWrapper, _byte_of_symbol, load_tokenizer

    table = _byte_of_symbol()
    assert sorted(table.values()) == list(range(256)) and table["A"] == 65 and table["Ġ"] == 32
    tok = load_tokenizer(folder)
    det = tok.detokenizer
    assert det._token_bytes is not None
    assert det._token_bytes(0) == b"<|endoftext|>"  # an added token is its own text
    words = Tokenizer(models.WordLevel({"[UNK]": 0, "fox": 1, "dog": 2, "\n": 3}, unk_token="[UNK]"))
    words.pre_tokenizer = pre_tokenizers.Whitespace()
    plain_tok = TokenizerWrapper(words)
    det = plain_tok.detokenizer
    assert det._token_bytes is None
    for t in (1, 2, 1):
        det.add_token(t)
    det.finalize()
    assert det.text == plain_tok.decode([1, 2, 1]) and det.tokens == [1, 2, 1]
