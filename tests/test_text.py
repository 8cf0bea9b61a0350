"""Text at the engine's edges (CPU, torch stand-ins for the kernels): prompts as text through the model
folder's tokenizer.json, the text of the generated tokens piece by piece, stop strings. The tokenizers are
made here: a word-level one and a byte-level one without merges, in which a letter beyond ASCII is two
tokens, so that a piece can end in the middle of a letter."""
import os

import pytest

from helpers import TINY, make_model_folder
from torch_ops import TorchOps

from lmsf_amd.engine import EngineArgs, LLMEngine
from lmsf_amd.engine.detokenizer import IncrementalDetokenizer, Tokenizer, load_tokenizer
from lmsf_amd.engine.llm_engine import check_stop
from lmsf_amd.engine.sequence import Sequence, SequenceState
from lmsf_amd.sampling import SamplingParams

tokenizers = pytest.importorskip("tokenizers")


def write_word_tokenizer(folder, n_words=250):
    from tokenizers import Tokenizer as T, decoders, models, pre_tokenizers
    vocab = {"<unk>": 0, "<s>": 1, "</s>": 2}
    for w in ["to", "be", "or", "not", ",", "that", "is", "the", "question", "."]:
        vocab[w] = len(vocab)
    while len(vocab) < n_words:
        vocab["w%d" % len(vocab)] = len(vocab)
    tok = T(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.decoder = decoders.WordPiece(prefix="##", cleanup=False)
    path = os.path.join(folder, "tokenizer.json")
    tok.save(path)
    return path


def write_byte_tokenizer(folder):
    from tokenizers import Tokenizer as T, decoders, models, pre_tokenizers
    alphabet = sorted(pre_tokenizers.ByteLevel.alphabet())
    vocab = {ch: i for i, ch in enumerate(alphabet)}
    tok = T(models.BPE(vocab=vocab, merges=[]))
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
    tok.decoder = decoders.ByteLevel()
    path = os.path.join(folder, "tokenizer.json")
    tok.save(path)
    return path


def pieces_of(tok, prompt_ids, out_ids):
    d = IncrementalDetokenizer(tok, len(prompt_ids))
    return [d.step(prompt_ids + out_ids[:i + 1]) for i in range(len(out_ids))]


def test_pieces_add_up_to_the_decoded_text(tmp_path):
    tok = Tokenizer(write_word_tokenizer(str(tmp_path)))
    prompt = tok.encode("to be or not")
    out = tok.encode("to be , that is the question .")
    pieces = pieces_of(tok, prompt, out)
    assert "".join(pieces) == " " + tok.decode(out)          # the first piece keeps the blank after the prompt
    assert all(p for p in pieces)
    # without a prompt before it the first piece has no blank
    assert "".join(pieces_of(tok, [], out)) == tok.decode(out)


def test_a_piece_waits_for_the_rest_of_a_letter(tmp_path):
    tok = Tokenizer(write_byte_tokenizer(str(tmp_path)))
    text = "café naïve — 東京"
    out = tok.encode(text)
    assert len(out) > len(text)                                # letters of several tokens
    pieces = pieces_of(tok, tok.encode("x "), out)
    assert "".join(pieces) == text and all("�" not in p for p in pieces)
    assert "" in pieces                                        # held back at least once
    assert load_tokenizer(str(tmp_path)) is not None and load_tokenizer(str(tmp_path / "nothing")) is None
    assert load_tokenizer(None) is None


def test_stop_strings_in_the_reference_order():
    def seq_with(text, params, out_ids=(5,), prompt=(1, 2)):
        s = Sequence("r", list(prompt), params, 0, 0, output_token_ids=list(out_ids))
        s.output_text = text
        return s
    s = seq_with("to be or", SamplingParams(stop=["or", "zz"]))
    check_stop(s, 100, {2})
    assert s.state == SequenceState.FINISHED_STOPPED and s.output_text == "to be " and s.state.finish_reason == "stop"
    s = seq_with("to be or", SamplingParams(stop="or", include_stop_str_in_output=True))
    check_stop(s, 100, {2})
    assert s.state == SequenceState.FINISHED_STOPPED and s.output_text == "to be or"
    # only at the end of the text, as in the reference
    s = seq_with("or to be", SamplingParams(stop=["or"]))
    check_stop(s, 100, {2})
    assert s.state == SequenceState.WAITING
    # a stop string comes before the other rules: the same step would also have hit max_tokens and EOS
    s = seq_with("x.", SamplingParams(stop=["."], max_tokens=1), out_ids=(2,))
    check_stop(s, 100, {2})
    assert s.state == SequenceState.FINISHED_STOPPED and s.output_text == "x"
    s = seq_with("x", SamplingParams(max_tokens=1), out_ids=(7,))
    check_stop(s, 100, {2})
    assert s.state == SequenceState.FINISHED_LENGTH_CAPPED
    for bad in ([""], [3]):
        with pytest.raises(ValueError):
            SamplingParams(stop=bad)


def make_engine(tmp_path, with_tokenizer=True, **kw):
    folder, cfg = make_model_folder(tmp_path, "A")
    if with_tokenizer:
        write_word_tokenizer(folder, n_words=cfg.vocab_size)
    args = EngineArgs(model=folder, dtype="float32", block_size=TINY["A"][2], device="cpu",
                      num_gpu_blocks_override=64, max_num_seqs=8, **kw)
    return LLMEngine(args, ops=TorchOps()), folder, cfg


def run(engine):
    done, streamed = {}, {}
    while engine.has_unfinished_requests():
        for out in engine.step():
            streamed[out.request_id] = streamed.get(out.request_id, "") + out.outputs[0].latest_text
            if out.finished:
                done[out.request_id] = out
    return done, streamed


def test_text_in_text_out(tmp_path):
    engine, folder, cfg = make_engine(tmp_path)
    tok = engine.tokenizer
    greedy = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    engine.add_request("t", "to be or not to be ,", greedy)
    engine.add_request("i", tok.encode("to be or not to be ,"), SamplingParams(**vars(greedy)))
    engine.add_request("o", "ignored text", SamplingParams(**vars(greedy)), prompt_token_ids=tok.encode("to be or not to be ,"))
    done, streamed = run(engine)
    t, i, o = done["t"], done["i"], done["o"]
    assert t.prompt == "to be or not to be ," and i.prompt is None and o.prompt == "ignored text"
    assert t.prompt_token_ids == i.prompt_token_ids == o.prompt_token_ids == tok.encode("to be or not to be ,")
    assert t.outputs[0].token_ids == i.outputs[0].token_ids == o.outputs[0].token_ids
    assert t.outputs[0].text == " " + tok.decode(t.outputs[0].token_ids) and streamed["t"] == t.outputs[0].text
    # a stop string: the text of the third generated token ends the request there, cut off or kept
    words = t.outputs[0].text.split()
    stop = words[2]
    first = words.index(stop)
    engine.add_request("s", "to be or not to be ,", SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True, stop=[stop]))
    engine.add_request("k", "to be or not to be ,", SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True, stop=[stop],
                                                                   include_stop_str_in_output=True))
    done, streamed = run(engine)
    s, k = done["s"].outputs[0], done["k"].outputs[0]
    assert s.finish_reason == k.finish_reason == "stop"
    assert s.token_ids == k.token_ids == t.outputs[0].token_ids[:first + 1]
    assert k.text == " " + " ".join(words[:first + 1]) and s.text == k.text[:-len(stop)]
    assert streamed["s"] == s.text and streamed["k"] == k.text
    engine.core.storage.manager.check_invariants()
    assert engine.core.storage.manager.num_free_pages(0) == 64


def test_without_a_tokenizer_text_is_refused(tmp_path):
    engine, folder, cfg = make_engine(tmp_path, with_tokenizer=False)
    assert engine.tokenizer is None
    with pytest.raises(ValueError, match="tokenizer.json"):
        engine.add_request("t", "to be", None)
    with pytest.raises(ValueError, match="tokenizer.json"):
        engine.add_request("s", [1, 2, 3], SamplingParams(stop=["x"]))
    engine.add_request("i", [1, 2, 3], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))
    done, _ = run(engine)
    assert done["i"].outputs[0].text == "" and len(done["i"].outputs[0].token_ids) == 2
    # and an engine told to skip the tokenizer does not load the one that is there
    engine2, _, _ = make_engine(tmp_path / "two", skip_tokenizer_init=True)
    assert engine2.tokenizer is None
