"""Autoregressive batch engine for the sequence-mixer models (models/seqmix.py).

Where the speculation engines run ONE conversation through a draft tree and a tree-masked verify, this engine serves
MANY requests with no draft at all -- a recurrent state cannot be rolled back the way a KV slot is recycled, so these models
are decoded token by token -- and gets its throughput from batching instead: every step is one ragged forward over all
running requests.

Scheduling is static batching: when nothing runs, queued requests are admitted first come first served while sequence
slots and cache pages last, and their prompts are prefilled together in one step; from then on every step decodes one token
for each of them; a request that finishes gives its pages and slot back at once; the queue is looked at again when the
batch has drained.  One function, ``run_step``, executes a step for both the scheduler and callers that bring their own
tokens (trace replay): it owns the page / slot bookkeeping and calls the model's ragged forward.

It keeps the engine surface (speculation/base.py) so the front-ends work unchanged: ``prefill`` / ``append`` /
``speculative_decoding`` drive one conversation (a tree of size one: ``build_tree`` has nothing to build, ``verify`` is a
plain decode step), ``generate`` / ``generate_stream`` answer one API request, ``generate_batch`` many.
Sampling uses the same device kernels as the speculation engines (arg-max, or penalty / top-k / temperature / top-p).
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

import torch

from .. import _lib
from ..logging_config import setup_logger
from ..models import AutoModelLM
from ..utils import TextColors
from .base import BaseEngine
from .speculation_utils import IdTokenizer, is_sentence_complete_regex

logger = setup_logger()


@dataclass
class Request:
    id: object
    prompt: list
    max_new_tokens: int
    generated: list = field(default_factory=list)
    done: bool = False
    pending: int | None = None          # sampled, not yet fed through the model
    recorded: int = 0                   # tokens written to the device-side history of its slot


class BatchEngine(BaseEngine):
    NEEDS_DRAFT = False
    CHAT = "__chat__"

    def __init__(self, draft_model_name=None, target_model_name=None, dtype=torch.bfloat16, device: str = "cuda:0", **kwargs):
        super().__init__()
        self.target_model_name, self.dtype, self.device = target_model_name, dtype, device
        self.max_length = kwargs.pop("max_length", 8192)
        self.max_batch = kwargs.pop("max_batch", 8)
        self.max_tokens = kwargs.pop("max_tokens", None)
        self.page_size = kwargs.pop("page_size", 64)
        self.stop_distance = kwargs.pop("stop_distance", 32)
        self.temperature = kwargs.pop("temperature", 0.0)
        self.topp = kwargs.pop("topp", 0.9)
        self.topk = kwargs.pop("topk", 32)
        self.repetition_penalty = kwargs.pop("repetition_penalty", 1.0)
        self.seed = kwargs.pop("seed", 0)
        self._target_model = kwargs.pop("target_model_obj", None)
        self._tokenizer = kwargs.pop("tokenizer", None)
        self.config = kwargs

    # ------------------------------------------------------------------ setup
    def initialize(self):
        if self._target_model is None:
            self.target_model = AutoModelLM.from_pretrained(
                model_name=self.target_model_name, batch_size=self.max_batch, max_length=self.max_length, device=self.device,
                dtype=self.dtype, max_tokens=self.max_tokens, page_size=self.page_size)
            self.target_model.alloc()
        else:
            self.target_model = self._target_model
        if not hasattr(self.target_model, "forward_batch"):
            raise ValueError("the batch engine serves sequence-mixer models (models/seqmix.py); tree-decoded models run on "
                             "the static / dynamic speculation engines")
        m = self.target_model
        self.max_length, self.max_batch = m.max_length, m.batch_size
        self.vocab_size = m.config.vocab_size
        self.eos_tokens = list(m.eos_tokens)
        if self._tokenizer is not None:
            self.tokenizer = self._tokenizer
        else:
            try:
                from transformers import AutoTokenizer
                self.tokenizer = AutoTokenizer.from_pretrained(self.target_model_name, local_files_only=True)
            except Exception as e:
                logger.warning(f"NO TOKENIZER for '{self.target_model_name}' ({type(e).__name__}): falling back to the "
                               "id tokenizer -- text is read and written as space-separated token ids")
                self.tokenizer = IdTokenizer()
        dev = self.device
        self.sampled = torch.zeros(self.max_batch, dtype=torch.int32, device=dev)
        self.rng_state = torch.tensor([self.seed], dtype=torch.int64, device=dev)
        self.step_count = torch.zeros(1, dtype=torch.int32, device=dev)
        self.history = torch.zeros(self.max_batch, self.max_length + 1, dtype=torch.int32, device=dev)   # per slot: its tokens
        self.hist_len = torch.zeros(self.max_batch, dtype=torch.int32, device=dev)
        self.queue, self.running, self.finished = deque(), [], {}
        self._next_id = 0
        self.num_nodes = 0

    # ------------------------------------------------------------------ the step function
    @torch.inference_mode()
    def run_step(self, entries, end=()):
        """One step.  entries: [(request id, next tokens, indices whose logits are wanted)]; a request seen for the first
        time gets a sequence slot, `end` lists the requests whose pages, state and slot are given back after the step.
        Returns fp32 logits [rows wanted, V] in the order of the entries (a workspace view, valid until the next step)."""
        m = self.target_model
        cache = m.kv_cache
        parts, want = [], []
        for rid, toks, w in entries:
            if rid not in cache.seqs:
                m.open(rid)
            if len(toks) == 0:                  # a request that brings nothing this step only keeps (or takes) its slot
                continue
            parts.append((rid, toks))
            want.append(list(w))
        logits = m.forward_batch(parts, want=want) if parts else None
        for rid in end:
            if rid in cache.seqs:
                m.close(rid)
        return logits

    def _greedy(self):
        return self.temperature < 0.05 and not (self.repetition_penalty > 1.01)

    def _sample(self, logits, reqs):
        """one token per logits row (row i belongs to reqs[i]) -> list of ints"""
        R = logits.shape[0]
        out = self.sampled[:R]
        if self._greedy():
            _lib.seq_call("umb_argmax_rows", out, logits, R, self.vocab_size)
        else:
            k = min(int(self.topk), self.vocab_size)
            self.step_count += 1
            if self.repetition_penalty > 1.01:
                for i, r in enumerate(reqs):          # every request is penalised over its own history
                    slot = self.target_model.kv_cache.slot(r.id)
                    _lib.seq_call("umb_sample_rows", out[i:i + 1], logits[i:i + 1], 1, self.vocab_size, self.history[slot],
                                  self.hist_len[slot:slot + 1], float(self.repetition_penalty), float(self.temperature), k,
                                  float(self.topp), self.rng_state, 0, None, None)
            else:
                _lib.seq_call("umb_sample_rows", out, logits, R, self.vocab_size, self.history[0], self.step_count, 1.0,
                              float(self.temperature), k, float(self.topp), self.rng_state, 0, None, None)
        return out.tolist()

    def _record(self, req, tokens):
        """append tokens to the request's device-side history (read by the repetition penalty)"""
        if not (self.repetition_penalty > 1.01):
            return
        slot = self.target_model.kv_cache.slot(req.id)
        n = req.recorded
        t = torch.tensor(tokens, dtype=torch.int32, device=self.device)
        self.history[slot, n:n + len(tokens)] = t
        req.recorded = n + len(tokens)
        self.hist_len[slot] = req.recorded - 1             # the kernel reads indices 0 .. n inclusive

    # ------------------------------------------------------------------ scheduler
    def submit(self, input_ids, max_new_tokens: int = 128, request_id=None):
        ids = [int(t) for t in (input_ids.reshape(-1).tolist() if isinstance(input_ids, torch.Tensor) else input_ids)]
        if not ids:
            raise ValueError("a request needs at least one prompt token")
        if len(ids) + max_new_tokens > self.max_length:
            raise ValueError(f"prompt ({len(ids)}) + max_new_tokens ({max_new_tokens}) exceeds max_length {self.max_length}")
        if request_id is None:
            request_id, self._next_id = self._next_id, self._next_id + 1
        self.queue.append(Request(request_id, ids, int(max_new_tokens)))
        return request_id

    def _admit(self):
        """static batching: called only when nothing runs; first come first served while slots and pages last"""
        cache = self.target_model.kv_cache
        budget = len(cache.free_pages)
        while self.queue and len(self.running) < self.max_batch and len(cache.free_slots) > len(self.running):
            r = self.queue[0]
            need = (len(r.prompt) + r.max_new_tokens + cache.page - 1) // cache.page
            if need > budget:
                if not self.running:
                    raise RuntimeError(f"request {r.id!r} needs {need} cache pages, the cache has {budget} free")
                break
            budget -= need
            self.running.append(self.queue.popleft())

    def _retire(self, r):
        r.done = True
        self.finished[r.id] = r
        self.running.remove(r)

    @torch.inference_mode()
    def step(self) -> bool:
        """One scheduler step (prefill of a fresh batch, or one decoded token for every running request).  Returns
        whether anything is left to do."""
        if not self.running:
            self._admit()
            if not self.running:
                return False
            batch = list(self.running)
            entries = [(r.id, r.prompt, [len(r.prompt) - 1]) for r in batch]
            for r in batch:
                self.target_model.open(r.id)
                self._record(r, r.prompt)
        else:
            batch = list(self.running)
            entries = [(r.id, [r.pending], [0]) for r in batch]
        logits = self.run_step(entries)
        new = self._sample(logits, batch)
        end = []
        for r, tok in zip(batch, new):
            r.generated.append(tok)
            r.pending = tok
            self._record(r, [tok])
            if len(r.generated) >= r.max_new_tokens or tok in self.eos_tokens:
                end.append(r)
        for r in end:
            self.target_model.close(r.id)
            self._retire(r)
        return bool(self.running or self.queue)

    @torch.inference_mode()
    def generate_batch(self, prompts, max_new_tokens: int = 128):
        """prompts: list of token-id lists -> list of generated token-id lists (greedy or sampled per the engine's knobs)"""
        ids = [self.submit(p, max_new_tokens) for p in prompts]
        while self.step():
            pass
        return [self.finished.pop(i).generated for i in ids]

    # ------------------------------------------------------------------ one conversation (engine surface)
    def prefill(self, text: str):
        return self._prefill(self.tokenizer.encode(text, return_tensors="pt"))

    def append(self, text: str):
        return self._append(self.tokenizer.encode(text, return_tensors="pt")[:, 1:])

    def _feed_chat(self, ids):
        cache = self.target_model.kv_cache
        held = cache.length(self.CHAT) if self.CHAT in cache.seqs else 0
        if held + len(ids) + self.stop_distance >= self.max_length or \
                (self.CHAT in cache.seqs and not cache.can_extend(self.CHAT, len(ids) + self.stop_distance)):
            return False
        logits = self.run_step([(self.CHAT, ids, [len(ids) - 1])])
        self._chat.prompt.extend(ids)
        self._record(self._chat, ids)
        self._chat.pending = self._sample(logits, [self._chat])[0]
        self.num_nodes = cache.length(self.CHAT)
        return True

    @torch.inference_mode()
    def _prefill(self, input_ids):
        if self.CHAT not in self.target_model.kv_cache.seqs:
            self._chat = Request(self.CHAT, [], 0)
        return self._feed_chat([int(t) for t in input_ids.reshape(-1).tolist()])

    @torch.inference_mode()
    def _append(self, input_ids):
        assert getattr(self, "_chat", None) is not None, "append() follows prefill()"
        ids = [int(t) for t in input_ids.reshape(-1).tolist()]
        return self._feed_chat([self._chat.pending] + ids)          # the pending token becomes context

    def build_tree(self):
        """nothing to draft: the 'tree' of an autoregressive step is its root"""

    @torch.inference_mode()
    def verify(self) -> bool:
        """feed the pending token, sample the next; returns continue_generation"""
        c = self._chat
        logits = self.run_step([(self.CHAT, [c.pending], [0])])
        c.generated.append(c.pending)
        self._record(c, [c.pending])
        c.pending = self._sample(logits, [c])[0]
        self.num_nodes = self.target_model.kv_cache.length(self.CHAT)
        return c.generated[-1] not in self.eos_tokens

    def validate_status(self):
        cache = self.target_model.kv_cache
        return self.num_nodes + self.stop_distance < self.max_length and \
            (self.CHAT not in cache.seqs or cache.can_extend(self.CHAT, 1))

    def _decode_words(self, ids):
        return (self.tokenizer.decode(ids, skip_special_tokens=True, clean_up_tokenization_spaces=False,
                                      spaces_between_special_tokens=False).strip().split(" "))

    @torch.inference_mode()
    def speculative_decoding(self, max_new_tokens=128):
        max_new_tokens = max(max_new_tokens, self.stop_distance)
        torch.cuda.synchronize()
        t1 = time.time()
        steps, decode, ids, pos, words = 0, True, [], 0, [""]
        while decode and self.validate_status():
            decode = self.verify()
            steps += 1
            ids.append(self._chat.generated[-1])
            words = self._decode_words(ids)
            now = len(words) - 1
            if now > pos:
                print(" ".join(words[pos:now]), end=" ", flush=True)
                pos = now
            if (is_sentence_complete_regex(words[-1]) and steps >= max_new_tokens - self.stop_distance) or steps >= max_new_tokens:
                decode = False
        print(" ".join(words[pos:]), flush=True)
        torch.cuda.synchronize()
        t2 = time.time()
        logger.info(TextColors.colorize("Avg Accept Tokens {:.2f} | TPOT {:.2f} ms ".format(1.0, 1000 * (t2 - t1) / max(steps, 1)),
                                        "magenta"))
        return steps + 1, (t2 - t1), steps

    # ------------------------------------------------------------------ API requests
    def update_generation_args(self, **generation_args):
        self.temperature = generation_args.pop("temperature", self.temperature)
        self.topp = generation_args.pop("topp", self.topp)
        self.repetition_penalty = generation_args.pop("repetition_penalty", self.repetition_penalty)
        self.topk = generation_args.pop("topk", self.topk)

    def manual_seed(self, seed: int):
        self.seed = seed
        self.rng_state.fill_(seed)

    def _request_ids(self, api_args):
        input_ids = api_args.get("input_ids", None)
        if input_ids is None:
            context = api_args.get("context", None)
            if not context:
                return None
            return self.tokenizer.encode(context, return_tensors="pt").reshape(-1).tolist()
        return list(input_ids)

    @torch.inference_mode()
    def generate(self, **api_args):
        self.update_generation_args(**api_args)
        ids, n = self._request_ids(api_args), api_args.get("max_new_tokens", 128)
        if not ids or n == 0 or len(ids) + n > self.max_length:
            api_args.update(generated_text="", generated_tokens=[], avg_accept_tokens=0, time_per_output_token=0)
            return api_args
        torch.cuda.synchronize()
        t1 = time.time()
        toks = self.generate_batch([ids], n)[0]
        torch.cuda.synchronize()
        t2 = time.time()
        api_args["generated_text"] = self.tokenizer.decode(toks, skip_special_tokens=True, clean_up_tokenization_spaces=False)
        api_args["generated_tokens"] = toks
        api_args["avg_accept_tokens"] = 1.0
        api_args["time_per_output_token"] = 1000 * (t2 - t1) / max(len(toks), 1)
        return api_args

    @torch.inference_mode()
    def generate_stream(self, **api_args):
        self.update_generation_args(**api_args)
        ids, n = self._request_ids(api_args), api_args.get("max_new_tokens", 128)
        if not ids or n == 0:
            return
        if len(ids) + n > self.max_length:
            yield "Exceeding reserved allowed context length", "Exceeding reserved allowed context length"
            return
        rid = self.submit(ids, n)
        t1, text = time.time(), ""
        while self.step():
            r = next((q for q in self.running if q.id == rid), None)
            if r is None:
                break
            text = " ".join(self._decode_words(r.generated))
            yield text, "Output Tokens {} | TPOT {:.2f} ms ".format(len(r.generated), 1000 * (time.time() - t1) / len(r.generated))
        r = self.finished.pop(rid)
        yield " ".join(self._decode_words(r.generated)), "Output Tokens {} | TPOT {:.2f} ms ".format(
            len(r.generated), 1000 * (time.time() - t1) / max(len(r.generated), 1))

    @torch.inference_mode()
    def reset(self):
        self.target_model.clear()
        self.queue.clear()
        self.running.clear()
        self.finished.clear()
        self._chat = None
        self.num_nodes = 0
        self.hist_len.zero_()
