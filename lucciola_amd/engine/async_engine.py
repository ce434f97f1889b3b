"""An asynchronous front in the manner of the reference's ``AsyncEngine``
(include/async_engine.h:22-35, src/async_engine.cc): construct with ``(model_path,
max_blocks=0, block_size=16)``, submit with ``generate_async(prompt, max_new_tokens,
callback)`` from any thread, a background thread runs the engine loop and calls
``callback(token, is_finished)`` for every generated token, ``stop()`` ends it.

The engine works on token ids.  A prompt may be a list of ids (the callback then gets
``(token id, is_finished)``) or, where the model folder holds a ``vocab.json``, a string as in
the reference: it is put into the reference's chat format (src/async_engine.cc:82-106) and the
callback gets ``(text, is_finished)``.  The table of live requests is touched only under the
lock (the reference's loop reads it without, src/async_engine.cc:140-153 against :42-48).
"""
from __future__ import annotations

import threading
from typing import Callable, Dict, List, Optional, Sequence as Seq, Tuple, Union

from ..config.engine_config import EngineConfig
from ..sampling.sampler import SamplingParams
from ..text.vocab_tokenizer import ChatFormat, VocabTokenizer, find_vocab
from .llm_engine import LLMEngine


class AsyncEngine:
    def __init__(self, model_path: str, max_blocks: int = 0, block_size: int = 16,
                 dtype="bfloat16", max_tokens_per_step: int = 2048, max_seqs: int = 256,
                 device: str = "cuda:0", engine: Optional[LLMEngine] = None,
                 tokenizer: Optional[VocabTokenizer] = None,
                 chat_format: Optional[ChatFormat] = ChatFormat()):
        if engine is None:
            cfg = EngineConfig(dtype=dtype, block_size=block_size, max_blocks=max_blocks,
                               max_tokens_per_step=max_tokens_per_step, max_seqs=max_seqs,
                               device=device)
            engine = LLMEngine.from_folder(model_path, cfg)
        self.engine = engine
        self.tokenizer = tokenizer if tokenizer is not None or not model_path else find_vocab(model_path)
        self.chat_format = chat_format        # None: text prompts are encoded as they are
        self._mu = threading.Lock()
        self._cv = threading.Condition(self._mu)
        self._stop = False
        self._pending: List[Tuple[int, List[int], SamplingParams]] = []
        self._callbacks: Dict[int, Callable[[int, bool], None]] = {}
        self._engine_ids: Dict[int, int] = {}
        self._aborts: List[int] = []
        self._next_req_id = 1
        self._error: Optional[BaseException] = None
        self._thread = threading.Thread(target=self._engine_loop, name="lucciola-engine", daemon=True)
        self._thread.start()

    def generate_async(self, prompt: Union[str, Seq[int]], max_new_tokens: int,
                       callback: Callable[[Union[int, str], bool], None], temperature: float = 0.0,
                       seed: int = 0) -> int:
        """Submit a request; returns its id.  ``callback(token_id, is_finished)`` runs on the
        engine thread for every generated token; for a prompt given as text it is
        ``callback(text, is_finished)`` with the text that the token adds."""
        params = SamplingParams(max_new_tokens=max_new_tokens, temperature=temperature, seed=seed)
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a vocab.json in the model folder")
            prompt = (self.chat_format.prompt(self.tokenizer, prompt) if self.chat_format
                      else self.tokenizer.encode(prompt))
            callback = self._as_text(callback)
        with self._cv:
            if self._error is not None:
                raise RuntimeError("the engine loop has failed") from self._error
            req_id = self._next_req_id
            self._next_req_id += 1
            self._callbacks[req_id] = callback
            self._pending.append((req_id, [int(t) for t in prompt], params))
            self._cv.notify()
        return req_id

    def _as_text(self, text_callback: Callable[[str, bool], None]) -> Callable[[int, bool], None]:
        text = self.tokenizer.stream()

        def on_token(token: int, finished: bool) -> None:
            # -1 stands for no token (the request was refused or ended early)
            text_callback(text.feed(token, finished) if token >= 0 else "", finished)
        return on_token

    def abort(self, req_id: int) -> None:
        """End a request: the engine thread frees what it holds and calls its callback once
        more with ``(-1, True)``.  (The reference has no way to end a request early.)"""
        with self._cv:
            self._aborts.append(req_id)
            self._cv.notify()

    def stop(self) -> None:
        with self._cv:
            if self._stop:
                return
            self._stop = True
            self._cv.notify_all()
        self._thread.join()

    def __del__(self):
        try:
            self.stop()
        except Exception:
            pass

    def _engine_loop(self) -> None:
        import torch
        eng = self.engine
        if eng.runner.device.type == "cuda":
            torch.cuda.set_device(eng.runner.device)
        try:
            while True:
                with self._cv:
                    while not self._stop and not self._pending and not self._aborts \
                            and not eng.has_unfinished_requests():
                        self._cv.wait()
                    if self._stop:
                        return
                    pending, self._pending = self._pending, []
                    aborts, self._aborts = self._aborts, []
                for req_id, prompt, params in pending:
                    try:
                        engine_id = eng.add_request(prompt, params)
                    except ValueError:
                        with self._mu:
                            cb = self._callbacks.pop(req_id, None)
                        if cb:
                            cb(-1, True)
                        continue
                    with self._mu:
                        self._engine_ids[engine_id] = req_id
                for req_id in aborts:
                    with self._mu:
                        engine_id = next((e for e, r in self._engine_ids.items() if r == req_id), None)
                        cb = self._callbacks.pop(req_id, None) if engine_id is not None else None
                        if engine_id is not None:
                            del self._engine_ids[engine_id]
                    if engine_id is not None:
                        eng.abort_request(engine_id)
                        eng.sequences.pop(engine_id, None)
                        if cb:
                            cb(-1, True)
                for out in eng.step():
                    with self._mu:
                        req_id = self._engine_ids.get(out.seq_id)
                        cb = self._callbacks.get(req_id)
                        if out.finished:
                            self._engine_ids.pop(out.seq_id, None)
                            self._callbacks.pop(req_id, None)
                    if out.finished:
                        eng.sequences.pop(out.seq_id, None)
                    if cb:
                        cb(out.token, out.finished)
        except BaseException as exc:  # surfaced at the next submit
            with self._mu:
                self._error = exc
            raise
