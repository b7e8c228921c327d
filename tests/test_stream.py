"""What a request emits: a stream that a reader task can await while the engine steps, and text that is made a token
at a time from a byte-level vocabulary, holding back the bytes of a character that is still split across tokens.
The situations are those of the reference's tests (tests/test_engine.py:57-83, 389-424 there); its tokenizer is a
downloaded one, so a small byte-level tokenizer is built here with the ``tokenizers`` package instead."""
import asyncio

import pytest
import torch

from llmserver_amd.engine import STREAM_END, ByteLevelText, ByteLevelVocabulary, Engine, RequestStatus, TokenStream, load_model
from llmserver_amd.engine.stream import BYTE_OF_CHARACTER
from helpers import model_folder
from test_scheduler_and_engine import Script
from torch_ops import TorchOps

tokenizers = pytest.importorskip("tokenizers")
TEXT = "Hello 👋, café. 你好!\n"


def byte_tokenizer(merges=(), special=("<|end|>",), added=()):
    """A byte-level BPE tokenizer whose base vocabulary is the 256 bytes (id = byte), then the merges, then added tokens."""
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    alphabet = sorted(BYTE_OF_CHARACTER, key=BYTE_OF_CHARACTER.get)
    vocab = {character: index for index, character in enumerate(alphabet)}
    for left, right in merges:
        vocab[left + right] = len(vocab)
    tokenizer = Tokenizer(models.BPE(vocab=vocab, merges=list(merges)))
    tokenizer.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)
    tokenizer.decoder = decoders.ByteLevel()
    tokenizer.add_special_tokens(list(special))
    tokenizer.add_tokens(list(added))
    return tokenizer


def test_the_byte_alphabet_is_the_library_s():
    from tokenizers import pre_tokenizers
    assert set(BYTE_OF_CHARACTER) == set(pre_tokenizers.ByteLevel.alphabet()) and len(BYTE_OF_CHARACTER) == 256
    assert sorted(BYTE_OF_CHARACTER.values()) == list(range(256))
    every_byte = bytes(range(256)).decode("latin-1") + TEXT          # as UTF-8 this runs through most byte values
    tokens = byte_tokenizer().encode(every_byte).tokens
    assert bytes(BYTE_OF_CHARACTER[token] for token in tokens) == every_byte.encode("utf-8")


def test_text_comes_out_a_token_at_a_time_and_split_characters_are_held_back():
    tokenizer = byte_tokenizer()
    ids = tokenizer.encode(TEXT).ids + [tokenizer.token_to_id("<|end|>")]
    text = ByteLevelText(ByteLevelVocabulary(tokenizer))
    pieces = [text.push(token) for token in ids]
    assert "".join(pieces) + text.finish() == tokenizer.decode(ids, skip_special_tokens=True) == TEXT
    assert "�" not in "".join(pieces)
    wave = TEXT.index("👋")
    assert pieces[wave:wave + 4] == ["", "", "", "👋"]              # four bytes, four tokens: the character appears with the last
    cut = ByteLevelText(ByteLevelVocabulary(tokenizer))
    assert [cut.push(token) for token in tokenizer.encode("é").ids[:1]] == [""] and cut.finish() == "�"   # a request that ends mid-character


def test_merged_tokens_added_words_and_special_tokens():
    tokenizer = byte_tokenizer(merges=[("c", "a"), ("ca", "f"), ("Ã", "©")], added=["<tool>"])
    ids = tokenizer.encode("café <tool> ok").ids
    assert len(ids) < len("café <tool> ok".encode()) and tokenizer.token_to_id("<tool>") in ids
    vocabulary = ByteLevelVocabulary(tokenizer)
    assert vocabulary.special_ids == {tokenizer.token_to_id("<|end|>")}
    text = ByteLevelText(vocabulary)
    assert "".join(text.push(token) for token in ids + [tokenizer.token_to_id("<|end|>")]) + text.finish() == "café <tool> ok"


def test_a_tokenizer_that_is_not_byte_level_is_not_taken():
    from tokenizers import Tokenizer, models
    assert ByteLevelVocabulary.of(Tokenizer(models.WordLevel({"a": 0, "[UNK]": 1}, unk_token="[UNK]"))) is None
    assert ByteLevelVocabulary.of(object()) is None
    assert ByteLevelVocabulary.of(byte_tokenizer()) is not None


# ---------------------------------------------------------------- the stream itself
def test_stream_serves_readers_with_and_without_a_loop():
    stream = TokenStream()
    with pytest.raises(asyncio.QueueEmpty):
        stream.get_nowait()
    stream.put_nowait(5)
    assert not stream.empty() and stream.get_nowait() == 5 and stream.empty()

    async def scenario():
        seen = []

        async def reader():
            async for item in stream:
                seen.append(item)

        task = asyncio.create_task(reader())
        await asyncio.sleep(0)                     # the reader waits: nothing has been put yet
        assert not seen and not task.done()
        for item in (1, 2):
            stream.put_nowait(item)
            await asyncio.sleep(0)
        assert seen == [1, 2]
        stream.put_nowait(STREAM_END)
        await asyncio.wait_for(task, 1)
        assert stream.ended and seen == [1, 2]
        # two readers, two items: nobody is left waiting
        stream.put_nowait("x")
        first, second = asyncio.create_task(stream.get()), asyncio.create_task(stream.get())
        await asyncio.sleep(0)
        stream.put_nowait("y")
        assert sorted(await asyncio.wait_for(asyncio.gather(first, second), 1)) == ["x", "y"]

    asyncio.run(scenario())


# ---------------------------------------------------------------- through the engine
def engine_with(script, tokenizer=None, case="A", **options):
    model = load_model(model_folder(case), "cpu", torch.float32)
    defaults = dict(max_new_tokens=3, max_batch_size=2, max_num_batched_tokens=4, kv_cache_num_blocks=16, kv_cache_block_size=2,
                    ignore_eos=False, ops=TorchOps())
    defaults.update(options)
    engine = Engine(model, tokenizer, **defaults)
    return engine, Script(model, script)


def test_engine_streams_text_that_equals_the_tokenizer_s_decoding():
    tokenizer = byte_tokenizer()
    end = tokenizer.token_to_id("<|end|>")
    ids = tokenizer.encode(TEXT).ids + [end]
    assert end == 256                                      # behind the 256 bytes: the model must have a larger vocabulary
    engine, _ = engine_with([[token] for token in ids], tokenizer, case="B", max_new_tokens=len(ids) + 5, max_batch_size=1)
    engine.eos_token_ids = {end}
    request = engine.add_request("Hi")
    assert request.prompt_token_ids == tokenizer.encode("Hi").ids
    while engine.step():
        pass
    pieces = request.output_queue.drain()
    assert pieces[-1] is STREAM_END and "".join(pieces[:-1]) == request.emitted_text == TEXT
    assert all(isinstance(piece, str) and piece for piece in pieces[:-1])
    assert request.generated_token_ids == ids and request.status == RequestStatus.FINISHED
    assert engine.completed_requests[request.request_id].output_text == TEXT


def test_stream_text_off_and_no_tokenizer_emit_token_ids_or_nothing():
    engine, _ = engine_with([[50], [51], [52]], None, max_batch_size=1)
    request = engine.add_request(None, [10])
    while engine.step():
        pass
    assert request.output_queue.drain() == [50, 51, 52, STREAM_END]
    engine, _ = engine_with([[50], [51], [52]], byte_tokenizer(), max_batch_size=1, stream_text=False)
    request = engine.add_request(None, [10])               # reference: tests/test_engine.py:176-184 (stream_text=False skips text)
    while engine.step():
        pass
    assert request.output_queue.drain() == [STREAM_END] and request.emitted_text == ""


def test_a_reader_task_gets_tokens_while_run_steps():
    """reference: tests/test_engine.py:389-405 there.  The reader awaits the stream; it is woken between steps, and sees
    the first request's second token before the request that arrived later has produced anything."""
    engine, script = engine_with([[50], [51], [60], [61]], max_new_tokens=2, max_batch_size=1)
    first = engine.add_request(None, [10])
    assert engine.step() and first.output_queue.get_nowait() == 50
    second = engine.add_request(None, [20])
    observed = {}

    async def reader():
        assert await first.output_queue.get() == 51
        observed["calls"] = len(script.calls)
        observed["second"] = list(second.generated_token_ids)
        assert await first.output_queue.get() is STREAM_END

    async def both():
        task = asyncio.create_task(reader())
        await asyncio.sleep(0)
        await asyncio.wait_for(asyncio.gather(task, engine.run()), timeout=5)

    asyncio.run(both())
    assert observed == {"calls": 2, "second": []}          # one place: the later request had not started when the reader ran
    assert second.generated_token_ids == [60, 61] and len(script.calls) == 4


def test_a_request_cancelled_between_steps_never_runs():
    """reference: tests/test_engine.py:407-424 there."""
    engine, script = engine_with([[50], [51]], max_new_tokens=2, max_batch_size=1)
    first = engine.add_request(None, [10])
    assert engine.step() and first.output_queue.get_nowait() == 50
    second = engine.add_request(None, [20])

    async def cancel_after_the_second_token():
        assert await first.output_queue.get() == 51
        assert engine.cancel_request(second.request_id)

    async def both():
        task = asyncio.create_task(cancel_after_the_second_token())
        await asyncio.sleep(0)
        await asyncio.wait_for(asyncio.gather(task, engine.run()), timeout=5)

    asyncio.run(both())
    assert second.status == RequestStatus.CANCELLED and second.generated_token_ids == []
    assert [call["requests"] for call in script.calls] == [[first.request_id]] * 2
    assert not engine.scheduler.running and not engine.kv_cache.requests
    assert second.output_queue.drain() == [STREAM_END]
