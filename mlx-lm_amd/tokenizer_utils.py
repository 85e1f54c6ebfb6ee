"""Optional tokenizer of a model folder, with a streaming detokenizer."""

import json
import os


class StreamingDetokenizer:
    """Turns a stream of token ids into text piece by piece.

    The contract of the reference's detokenizers (mlx_lm/tokenizer_utils.py:
    11-58): ``reset()``, ``add_token(id)``, ``finalize()``, then ``text`` is
    everything so far, ``last_segment`` what was added since it was last read,
    ``tokens`` the ids.  This one decodes the tokens since the last line break
    again for every token (the reference's ``NaiveStreamingDetokenizer``,
    mlx_lm/tokenizer_utils.py:61-112) and holds back a trailing incomplete
    character.
    """

    def __init__(self, decode):
        self._decode = decode
        self.reset()

    def reset(self):
        self.offset = 0
        self.tokens = []
        self._text = ""
        self._current = []
        self._current_text = ""

    def add_token(self, token):
        self._current.append(int(token))
        self.tokens.append(int(token))

    def finalize(self):
        self._text += self._decode(self._current)
        self._current = []
        self._current_text = ""

    @property
    def text(self):
        if self._current:
            self._current_text = self._decode(self._current)
            if self._current_text.endswith("�"):
                self._current_text = self._current_text[:-1]
        if self._current_text.endswith("\n"):
            self._text += self._current_text
            self._current = []
            self._current_text = ""
        return self._text + self._current_text

    @property
    def last_segment(self):
        text = self.text
        segment = text[self.offset :]
        self.offset = len(text)
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

    @property
    def detokenizer(self):
        return StreamingDetokenizer(self.decode)

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
