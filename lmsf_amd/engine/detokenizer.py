"""Text at the engine's edges: the model folder's tokenizer.json and the text of the tokens so far.

The reference loads ``<model>/tokenizer.json`` with the tokenizers library
(core/src/engine/llm_engine.rs:93-100), encodes a prompt with special tokens added (:147-149) and
after every sampled token decodes a window of the sequence's last tokens and appends what the new
token added (core/src/common/tokenizer.rs:30-78; the offsets live in the sequence,
llm_engine.rs:195-205). The same is done here with two changes: the window starts a few tokens
before the first generated one, so that the first piece keeps the blank a word-piece model puts
before it (the reference decodes the first new token alone), and the prompt is never decoded.
A piece that ends in an unfinished UTF-8 sequence is held back until the tokens that finish it
arrive (tokenizer.rs:62), as there.

Everything here is optional: an engine whose model folder has no tokenizer.json works on token ids.
"""
import os
from typing import List, Optional, Sequence

REPLACEMENT = "�"
WINDOW_BEFORE = 5   # tokens before the first generated one that the first window holds


class TokenizerError(RuntimeError):
    pass


class Tokenizer:
    """encode / decode of a tokenizer.json."""

    def __init__(self, path: str):
        try:
            import tokenizers
        except ImportError as e:   # pragma: no cover - the package is part of the image
            raise TokenizerError("%s needs the tokenizers package: %s" % (path, e)) from e
        try:
            self._tok = tokenizers.Tokenizer.from_file(path)
        except Exception as e:  # noqa: BLE001 - the library raises plain Exception
            raise TokenizerError("cannot load tokenizer %s: %s" % (path, e)) from e
        self.path = path

    @property
    def vocab_size(self) -> int:
        return self._tok.get_vocab_size(with_added_tokens=True)

    def encode(self, text: str, add_special_tokens: bool = True) -> List[int]:
        return list(self._tok.encode(text, add_special_tokens=add_special_tokens).ids)

    def decode(self, ids: Sequence[int], skip_special_tokens: bool = True) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=skip_special_tokens)


def load_tokenizer(model_dir: Optional[str]) -> Optional[Tokenizer]:
    """The tokenizer of a model folder, or None if the folder has no tokenizer.json."""
    if not model_dir:
        return None
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    return Tokenizer(path)


class IncrementalDetokenizer:
    """Text that each new token adds. ``prefix`` .. ``read`` are tokens whose text has been given out and
    that stay in the window as context; tokens from ``read`` on have not been given out yet."""

    def __init__(self, tokenizer: Tokenizer, prompt_len: int, skip_special_tokens: bool = True):
        self.tokenizer = tokenizer
        self.skip_special_tokens = skip_special_tokens
        self.prefix = max(prompt_len - WINDOW_BEFORE, 0)
        self.read = prompt_len

    def step(self, all_token_ids: Sequence[int]) -> str:
        """Call with prompt + generated ids after every new token; returns the text to append."""
        before = self.tokenizer.decode(all_token_ids[self.prefix:self.read], self.skip_special_tokens)
        now = self.tokenizer.decode(all_token_ids[self.prefix:], self.skip_special_tokens)
        if len(now) > len(before) and not now.endswith(REPLACEMENT):
            self.prefix, self.read = self.read, len(all_token_ids)
            return now[len(before):]
        return ""
