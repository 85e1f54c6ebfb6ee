"""Optional tokenizer of a model folder, with a streaming detokenizer."""

import json
import os


def _byte_of_symbol():
    """Byte-level BPE writes every byte as one printable character: the bytes that print
    (``!`` to ``~``, ``¡`` to ``¬``, ``®`` to ``ÿ``) as themselves, the other 68 as the
    characters from U+0100 on, in the order of the bytes.  Returns character -> byte."""
    keep = [*range(ord("!"), ord("~") + 1), *range(0xA1, 0xAD), *range(0xAE, 0x100)]
    table, extra = {}, 0
    for b in range(256):
        if b in keep:
            table[chr(b)] = b
        else:
            table[chr(256 + extra)] = b
            extra += 1
    return table


class StreamingDetokenizer:
    """Turns a stream of token ids into text piece by piece.

    The contract of the reference's detokenizers (mlx_lm/tokenizer_utils.py:
    11-58): ``reset()``, ``add_token(id)``, ``finalize()``, then ``text`` is
    everything so far, ``last_segment`` what was added since it was last read,
    ``tokens`` the ids.  For a byte-level BPE vocabulary (what the reference's
    ``BPEStreamingDetokenizer`` serves, mlx_lm/tokenizer_utils.py:157-250) a
    token is a fixed run of bytes: each token's bytes are looked up once, and
    an incremental UTF-8 decoder turns the stream of bytes into text, holding
    back a character whose bytes have not all come.  The cost of a token does
    not grow with the text.  Other vocabularies decode the tokens since the last
    line break again for every token.
    """

    def __init__(self, decode, token_bytes=None):
        self._decode = decode
        self._token_bytes = token_bytes  # id -> bytes for a byte-level vocabulary, else None
        self.reset()

    def reset(self):
        import codecs

        self.offset = 0
        self.tokens = []
        self._text = ""
        self._utf8 = codecs.getincrementaldecoder("utf-8")("replace")
        self._line = []  # (other vocabularies) the tokens since the last line break
        self._line_text = ""

    def add_token(self, token):
        token = int(token)
        self.tokens.append(token)
        if self._token_bytes is not None:
            self._text += self._utf8.decode(self._token_bytes(token))
            return
        self._line.append(token)
        shown = self._decode(self._line)
        if shown.endswith("\ufffd"):  # a character whose tokens have not all come
            shown = shown[:-1]
        if shown.endswith("\n"):
            self._text += shown
            self._line, shown = [], ""
        self._line_text = shown

    def finalize(self):
        if self._token_bytes is not None:
            self._text += self._utf8.decode(b"", final=True)
        elif self._line:
            self._text += self._decode(self._line)
            self._line, self._line_text = [], ""

    @property
    def text(self):
        return self._text + self._line_text

    @property
    def last_segment(self):
        text = self.text
        segment, self.offset = text[self.offset :], len(text)
        return segment


class TokenizerWrapper:
    """``encode``/``decode``, the set of end-of-sequence ids and a detokenizer.

    The surface of mlx_lm/tokenizer_utils.py:284-475 that generation uses,
    over a ``tokenizers.Tokenizer`` read from the folder's ``tokenizer.json``.
    """

    def __init__(self, tokenizer, eos_token_ids=None, bos_token=None, eos_token=None, chat_template=None):
        self._tokenizer = tokenizer
        self.eos_token_ids = set(eos_token_ids or [])
        self.bos_token = bos_token
        self.eos_token = eos_token
        self.chat_template = chat_template

    @property
    def has_chat_template(self):
        return self.chat_template is not None

    def apply_chat_template(self, messages, tokenize=True, add_generation_prompt=False,
                            continue_final_message=False, **template_kwargs):
        """Render ``messages`` (dicts with ``role`` and ``content``) with the folder's Jinja template.

        The template sees ``messages``, ``bos_token``, ``eos_token``,
        ``add_generation_prompt`` and whatever else is passed by keyword, as in
        mlx_lm/tokenizer_utils.py:332-343.  With ``continue_final_message`` the
        text ends where the last message's content ends, so that the model
        goes on writing that message.
        """
        if self.chat_template is None:
            raise ValueError("this tokenizer has no chat template")
        if continue_final_message and add_generation_prompt:
            raise ValueError("continue_final_message and add_generation_prompt exclude each other")
        from jinja2.sandbox import ImmutableSandboxedEnvironment

        def raise_exception(message):
            raise ValueError(message)

        env = ImmutableSandboxedEnvironment(trim_blocks=True, lstrip_blocks=True)
        env.globals["raise_exception"] = raise_exception
        text = env.from_string(self.chat_template).render(
            messages=messages, bos_token=self.bos_token or "", eos_token=self.eos_token or "",
            add_generation_prompt=add_generation_prompt, **template_kwargs)
        if continue_final_message:
            last = str(messages[-1]["content"]).strip()
            at = text.rfind(last)
            if at < 0:
                raise ValueError("the template does not show the last message's content")
            text = text[: at + len(last)]
        return self.encode(text, add_special_tokens=False) if tokenize else text

    def encode(self, text, add_special_tokens=True):
        return self._tokenizer.encode(text, add_special_tokens=add_special_tokens).ids

    def decode(self, ids, skip_special_tokens=False):
        return self._tokenizer.decode(list(ids), skip_special_tokens=skip_special_tokens)

    def add_eos_token(self, token):
        tid = None
        try:
            tid = int(token)
        except ValueError:
            tid = self._tokenizer.token_to_id(token)
        if tid is None:
            raise ValueError(f"'{token}' is not a token for this tokenizer")
        self.eos_token_ids.add(tid)

    def _byte_level_table(self):
        """``id -> bytes`` if the vocabulary is byte-level BPE (its decoder says so), else ``None``."""
        if not hasattr(self, "_bytes_of"):
            self._bytes_of = None
            spec = json.loads(self._tokenizer.to_str())
            decoder = spec.get("decoder") or {}
            kinds = {decoder.get("type")} | {d.get("type") for d in decoder.get("decoders", [])}
            if "ByteLevel" in kinds and kinds <= {"ByteLevel", None}:
                byte_of = _byte_of_symbol()
                added = {t["id"] for t in spec.get("added_tokens", [])}
                cache = {}

                def bytes_of(token):
                    b = cache.get(token)
                    if b is None:
                        piece = self._tokenizer.id_to_token(token) or ""
                        if token in added or any(ch not in byte_of for ch in piece):
                            b = piece.encode("utf-8")  # an added token is its own text
                        else:
                            b = bytes(byte_of[ch] for ch in piece)
                        cache[token] = b
                    return b

                self._bytes_of = bytes_of
        return self._bytes_of

    @property
    def detokenizer(self):
        return StreamingDetokenizer(self.decode, self._byte_level_table())

    @property
    def vocab_size(self):
        return self._tokenizer.get_vocab_size()


def load_tokenizer(model_path, eos_token_ids=None):
    """A ``TokenizerWrapper`` if the folder has ``tokenizer.json``, else ``None``.

    End-of-sequence ids come from the config (mlx_lm/utils.py:534-536), else
    from ``eos_token`` of ``tokenizer_config.json``.
    """
    path = os.path.join(model_path, "tokenizer.json")
    if not os.path.exists(path):
        return None
    from tokenizers import Tokenizer

    tok = Tokenizer.from_file(path)
    if isinstance(eos_token_ids, int):
        eos_token_ids = [eos_token_ids]
    eos = set(eos_token_ids or [])
    bos = eos_text = template = None
    cfg_path = os.path.join(model_path, "tokenizer_config.json")
    if os.path.exists(cfg_path):
        with open(cfg_path) as fh:
            cfg = json.load(fh)

        def as_text(v):
            return v.get("content") if isinstance(v, dict) else v

        bos = as_text(cfg.get("bos_token"))
        eos_text = as_text(cfg.get("eos_token"))
        template = cfg.get("chat_template")
        if not eos and eos_text is not None:
            tid = tok.token_to_id(eos_text)
            if tid is not None:
                eos.add(tid)
    jinja = os.path.join(model_path, "chat_template.jinja")
    if os.path.exists(jinja):
        with open(jinja) as fh:
            template = fh.read()
    return TokenizerWrapper(tok, eos, bos, eos_text, template if isinstance(template, str) else None)
