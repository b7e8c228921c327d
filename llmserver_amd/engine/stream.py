"""What a request emits on its way: a stream a reader task can await, and text made token by token.

The reference gives every request an ``asyncio.Queue`` that ends with a sentinel (utils/engine.py:25, 221, 312) and
turns byte-level tokens into text incrementally, holding back the bytes of a character that is still split across
tokens (``ByteLevelStreamDecoder``, utils/engine.py:29-44; its tests: tests/test_engine.py:57-83, 389-424).
:class:`TokenStream` serves readers with and without an event loop; :class:`ByteLevelText` is the incremental
decoder, made from the tokenizer's own vocabulary.
"""
from __future__ import annotations

import asyncio
import codecs
import collections
import json
from typing import Dict, Optional

STREAM_END = None      # what a stream ends with (utils/engine.py:25 in the reference)


class TokenStream:
    """What a request emits, in order: token ids or pieces of text, then :data:`STREAM_END`.

    The engine puts items in without waiting (``put_nowait``).  A reader in an event loop awaits :meth:`get`, or
    iterates with ``async for`` up to the end marker; a reader without a loop polls :meth:`get_nowait` or takes
    everything with :meth:`drain`.  The engine's ``run()`` yields to the loop after every step, which is when
    readers that were woken run."""

    def __init__(self):
        self._items = collections.deque()
        self._waiting = collections.deque()        # futures of readers that found the stream empty
        self.ended = False

    def put_nowait(self, item) -> None:
        self._items.append(item)
        if item is STREAM_END:
            self.ended = True
        while self._waiting:
            reader = self._waiting.popleft()
            if not reader.done():
                reader.set_result(None)
                break

    def get_nowait(self):
        if not self._items:
            raise asyncio.QueueEmpty("the stream holds nothing at the moment")
        return self._items.popleft()

    async def get(self):
        """The next item, waiting for the engine if there is none yet."""
        while not self._items:
            reader = asyncio.get_running_loop().create_future()
            self._waiting.append(reader)
            try:
                await reader
            except BaseException:
                reader.cancel()
                if self._items and self._waiting:      # pass a wake-up that came for this reader on to the next
                    follower = self._waiting.popleft()
                    if not follower.done():
                        follower.set_result(None)
                raise
        return self._items.popleft()

    def __aiter__(self):
        return self

    async def __anext__(self):
        item = await self.get()
        if item is STREAM_END:
            raise StopAsyncIteration
        return item

    def empty(self) -> bool:
        return not self._items

    def qsize(self) -> int:
        return len(self._items)

    def task_done(self) -> None:
        """Readers written for an ``asyncio.Queue`` may call this; nothing is counted here."""

    def drain(self) -> list:
        items = list(self._items)
        self._items.clear()
        return items


def _byte_alphabet() -> Dict[str, int]:
    """The character that stands for each byte in a byte-level BPE vocabulary.  Bytes that are printable, non-blank
    Latin-1 characters ('!' to '~', '¡' to '¬', '®' to 'ÿ') stand for themselves; the 68 others are written, in
    increasing order, as the code points 256, 257, ...  (so that no token of the vocabulary contains blanks or
    control characters)."""
    plain = set(range(ord("!"), ord("~") + 1)) | set(range(ord("¡"), ord("¬") + 1)) | set(range(ord("®"), ord("ÿ") + 1))
    alphabet, shifted = {}, 0
    for byte in range(256):
        if byte in plain:
            alphabet[chr(byte)] = byte
        else:
            alphabet[chr(256 + shifted)] = byte
            shifted += 1
    return alphabet


BYTE_OF_CHARACTER = _byte_alphabet()


def _tokenizer_core(tokenizer):
    """The ``tokenizers.Tokenizer`` inside whatever was passed (itself, or a wrapper that keeps it)."""
    for candidate in (tokenizer, getattr(tokenizer, "backend_tokenizer", None), getattr(tokenizer, "_tokenizer", None)):
        if candidate is not None and hasattr(candidate, "id_to_token") and hasattr(candidate, "to_str"):
            return candidate
    return None


def _mentions_byte_level(node) -> bool:
    if isinstance(node, dict):
        return node.get("type") == "ByteLevel" or any(_mentions_byte_level(value) for value in node.values())
    if isinstance(node, list):
        return any(_mentions_byte_level(value) for value in node)
    return False


class ByteLevelVocabulary:
    """What :class:`ByteLevelText` needs of a tokenizer, read once: each id's bytes, and the ids that are never text."""

    def __init__(self, tokenizer):
        core = _tokenizer_core(tokenizer)
        if core is None:
            raise ValueError("incremental text needs a tokenizers.Tokenizer (or a wrapper around one)")
        description = json.loads(core.to_str())
        if not _mentions_byte_level(description.get("decoder")):
            raise ValueError("the tokenizer does not decode byte-level tokens")
        self._core = core
        added = description.get("added_tokens") or []
        self.special_ids = {entry["id"] for entry in added if entry.get("special")}
        self._added_text = {entry["id"]: entry["content"] for entry in added if not entry.get("special")}
        self._bytes: Dict[int, bytes] = {}

    @classmethod
    def of(cls, tokenizer) -> Optional["ByteLevelVocabulary"]:
        try:
            return cls(tokenizer)
        except (ValueError, KeyError, TypeError):
            return None

    def token_bytes(self, token_id: int) -> bytes:
        found = self._bytes.get(token_id)
        if found is None:
            if token_id in self.special_ids:
                found = b""
            elif token_id in self._added_text:                 # added words are stored as they read, not in the byte alphabet
                found = self._added_text[token_id].encode("utf-8")
            else:
                token = self._core.id_to_token(token_id)
                if token is None:
                    found = b""
                else:
                    try:
                        found = bytes(BYTE_OF_CHARACTER[character] for character in token)
                    except KeyError:
                        found = token.encode("utf-8")
            self._bytes[token_id] = found
        return found


class ByteLevelText:
    """Text of one request, a token at a time: ``push`` returns the characters that the new token completes (possibly
    none, if it ends in the middle of a character), ``finish`` what is left when the request ends (a replacement
    character for bytes that never became one)."""

    def __init__(self, vocabulary: ByteLevelVocabulary):
        self.vocabulary = vocabulary
        self._utf8 = codecs.getincrementaldecoder("utf-8")("replace")

    def push(self, token_id: int) -> str:
        return self._utf8.decode(self.vocabulary.token_bytes(token_id))

    def finish(self) -> str:
        return self._utf8.decode(b"", final=True)
