"""The tokenizer wrapper, on a tiny SentencePiece model trained here on a few made-up sentences.

The reference's golden cases (data/golden/tokenizer_cases.json) are token ids of the real
TinyLlama tokenizer, whose model file is not in the reference: parity with those values is
unpinned here.  What is checked is the wrapper's own behaviour (src/tokenizer.cpp:63-129):
begin-of-sequence in front, round trip, refusal of ids outside the vocabulary and of folders
without a tokenizer."""
import os

import pytest

from tlie_amd import EngineError, ErrorCode
from tlie_amd.tokenizer import Tokenizer

sentencepiece = pytest.importorskip("sentencepiece")

SENTENCES = [
    "the cache keeps keys and values in pages", "a request holds a block table of its pages",
    "pages come back when a request ends", "the scheduler cuts prompts into portions",
    "decode steps run one token for every request", "the norm scales a row by its root mean square",
    "rotary positions turn pairs of a head by an angle", "the gate is passed through silu and multiplied by up",
    "logits are returned at the wanted places only", "greedy sampling takes the first maximum",
] * 8


@pytest.fixture(scope="module")
def model_dir(tmp_path_factory):
    folder = tmp_path_factory.mktemp("tokenizer")
    corpus = folder / "corpus.txt"
    corpus.write_text("\n".join(SENTENCES) + "\n", encoding="utf-8")
    sentencepiece.SentencePieceTrainer.train(input=str(corpus), model_prefix=str(folder / "tokenizer"), vocab_size=120,
                                             model_type="bpe", bos_id=1, eos_id=2, unk_id=0, pad_id=-1,
                                             minloglevel=2)
    assert os.path.isfile(folder / "tokenizer.model")
    return str(folder)


def test_begin_of_sequence_round_trip_and_refusals(model_dir, tmp_path):
    tokenizer = Tokenizer(model_dir)
    text = "the scheduler keeps pages"
    ids = tokenizer.encode(text)
    assert ids[0] == 1 and all(0 <= token < 120 for token in ids)            # BOS in front (src/tokenizer.cpp:103-105)
    assert tokenizer.encode(text, add_bos=False) == ids[1:]
    assert tokenizer.encode(text, add_eos=True)[-1] == 2
    assert tokenizer.encode(text.encode("utf-8")) == ids
    assert tokenizer.decode(ids) == text
    assert tokenizer.decode(ids[1:]) == text
    with pytest.raises(EngineError) as caught:
        tokenizer.decode([5, 120])
    assert caught.value.code == ErrorCode.TOKENIZER
    with pytest.raises(EngineError) as caught:
        tokenizer.encode(b"\xff\xfe broken")
    assert caught.value.code == ErrorCode.TOKENIZER
    with pytest.raises(EngineError) as caught:
        Tokenizer(str(tmp_path))                                              # a folder of random weights has none
    assert caught.value.code == ErrorCode.TOKENIZER
    (tmp_path / "tokenizer.model").write_bytes(b"this is no sentencepiece model")
    with pytest.raises(EngineError) as caught:
        Tokenizer(str(tmp_path))
    assert caught.value.code == ErrorCode.TOKENIZER
