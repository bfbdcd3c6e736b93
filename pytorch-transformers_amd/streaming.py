"""Streamers: objects that ``generate(..., streamer=...)`` hands the tokens to while it runs.

The interface is the reference's (src/transformers/generation/streamers.py:23-39): ``put(ids)`` receives the
prompt's ids first and then every new token, as a one-dimensional tensor (or ``[1, n]``); ``end()`` says that
generation is over.  ``TextStreamer`` turns them into text on standard output as soon as whole words exist
(:41-135), ``TextIteratorStreamer`` puts the same pieces of text into a queue for another thread to iterate
over (:162-228).  Both take one prompt per ``generate`` call, as in the reference (:87-88).
"""
from __future__ import annotations

import queue
from typing import Optional

# Code points written without spaces between words, so that every character may be shown as soon as it is there:
# the CJK unified ideographs with their extensions A to E and the two compatibility blocks (:137-159).
_UNSPACED = ((0x4E00, 0x9FFF), (0x3400, 0x4DBF), (0x20000, 0x2A6DF), (0x2A700, 0x2B73F), (0x2B740, 0x2B81F),
             (0x2B820, 0x2CEAF), (0xF900, 0xFAFF), (0x2F800, 0x2FA1F))


def _unspaced(ch: str) -> bool:
    cp = ord(ch)
    return any(lo <= cp <= hi for lo, hi in _UNSPACED)


class BaseStreamer:
    """What ``generate`` calls (src/transformers/generation/streamers.py:23-39)."""

    def put(self, value):
        raise NotImplementedError

    def end(self):
        raise NotImplementedError


class TextStreamer(BaseStreamer):
    """Prints the text of the tokens as whole words form (src/transformers/generation/streamers.py:41-135).

    The ids since the last line break are decoded together after every token, since a token's text may depend on
    its neighbours; of that text, what has not been shown yet is shown up to the last space (a word's last piece
    may still change it), all of it after a line break (which also starts the ids anew) or if it ends with a
    character of a script written without spaces.  ``skip_prompt``: the first ``put`` of a call, the prompt, is not
    shown.  ``decode_kwargs`` go to ``tokenizer.decode``.
    """

    def __init__(self, tokenizer, skip_prompt: bool = False, **decode_kwargs):
        self.tokenizer = tokenizer
        self.skip_prompt = skip_prompt
        self.decode_kwargs = decode_kwargs
        self._ids: list = []     # ids since the last line break
        self._shown = 0          # characters of their text that have been shown
        self._prompt_next = True

    def put(self, value):
        shape = getattr(value, "shape", None)
        if shape is not None and len(shape) > 1:
            if shape[0] > 1:
                raise ValueError("TextStreamer only supports batch size 1")
            value = value[0]
        if self._prompt_next:
            self._prompt_next = False
            if self.skip_prompt:
                return
        self._ids.extend(int(t) for t in (value.tolist() if hasattr(value, "tolist") else value))
        text = self.tokenizer.decode(self._ids, **self.decode_kwargs)
        if text.endswith("\n"):
            piece, self._ids, self._shown = text[self._shown:], [], 0
        elif text and _unspaced(text[-1]):
            piece = text[self._shown:]
            self._shown = len(text)
        else:
            piece = text[self._shown:text.rfind(" ") + 1]
            self._shown += len(piece)
        self.on_finalized_text(piece)

    def end(self):
        piece = ""
        if self._ids:
            piece = self.tokenizer.decode(self._ids, **self.decode_kwargs)[self._shown:]
        self._ids, self._shown, self._prompt_next = [], 0, True
        self.on_finalized_text(piece, stream_end=True)

    def on_finalized_text(self, text: str, stream_end: bool = False):
        """Where the text goes: standard output, with a line break at the end of the stream."""
        print(text, flush=True, end="\n" if stream_end else "")


class TextIteratorStreamer(TextStreamer):
    """The same pieces of text through a queue: iterate over the streamer in one thread while ``generate`` runs in
    another (src/transformers/generation/streamers.py:162-228).  ``timeout``: seconds that ``put`` into and ``get``
    out of the queue wait (None: for ever); the iteration ends with the stream."""

    _END = object()

    def __init__(self, tokenizer, skip_prompt: bool = False, timeout: Optional[float] = None, **decode_kwargs):
        super().__init__(tokenizer, skip_prompt, **decode_kwargs)
        self.text_queue: "queue.Queue" = queue.Queue()
        self.timeout = timeout

    def on_finalized_text(self, text: str, stream_end: bool = False):
        self.text_queue.put(text, timeout=self.timeout)
        if stream_end:
            self.text_queue.put(self._END, timeout=self.timeout)

    def __iter__(self):
        return self

    def __next__(self) -> str:
        piece = self.text_queue.get(timeout=self.timeout)
        if piece is self._END:
            raise StopIteration
        return piece
