"""Text to token ids and back, for model folders that carry a SentencePiece `tokenizer.model`.

reference: `Tokenizer` (src/tokenizer.cpp:63-129) wraps SentencePiece, refuses invalid UTF-8 and
ids out of range, and `Encode` puts the begin-of-sequence id in front by default (:103-105).
Token ids are this engine's primary input; a folder of random weights has no tokenizer, and asking
for text there is a `tokenizer_error`.
"""
from __future__ import annotations

import os

from .errors import EngineError, ErrorCode


class Tokenizer:
    def __init__(self, model_dir: str):
        path = os.path.join(model_dir, "tokenizer.model")
        if not os.path.isfile(path):
            raise EngineError(ErrorCode.TOKENIZER, f"{path} does not exist: give token ids instead of text")
        try:
            import sentencepiece
            self._model = sentencepiece.SentencePieceProcessor(model_file=path)
        except Exception as error:  # the library raises its own types
            raise EngineError(ErrorCode.TOKENIZER, f"unable to load {path}: {error}") from None

    def encode(self, text: str, add_bos: bool = True, add_eos: bool = False) -> list[int]:
        if isinstance(text, bytes):
            try:
                text = text.decode("utf-8")
            except UnicodeDecodeError:
                raise EngineError(ErrorCode.TOKENIZER, "the prompt is not valid UTF-8") from None
        ids = list(self._model.encode(text))
        if add_bos:
            ids = [self._model.bos_id()] + ids
        if add_eos:
            ids = ids + [self._model.eos_id()]
        return ids

    def decode(self, ids) -> str:
        size = self._model.get_piece_size()
        for token in ids:
            if not 0 <= int(token) < size:
                raise EngineError(ErrorCode.TOKENIZER, f"token id {token} is outside the tokenizer's vocabulary")
        return self._model.decode([int(token) for token in ids])
