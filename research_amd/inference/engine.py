"""Inference engine on the paged KV cache (reference: rollouts/rollouts/inference/engine.py).

The reference's engine has the queues, the scheduler call and the sampling, but
no KV cache yet: its ``_forward_batch`` (engine.py:218-250) feeds every
sequence's whole token list through the model each step, ``step`` hands the
scheduler a made-up block count (engine.py:147) and ``flush_cache`` is empty
(engine.py:195-198).  This engine keeps the same public surface
(``generate``, ``add_request``, ``step``, ``has_pending``, ``update_weights``,
``get_weight_version``, ``flush_cache``, ``shutdown``) and fills those gaps:

* ``step`` = schedule (with the allocator's real free-block count) ->
  allocate / extend blocks -> build contexts -> one batched model forward for
  the prefills and one for the decodes, through ``Attention`` layers on the HIP
  backend -> ``sample_with_logprobs``.
* Prefill is chunked over whatever prefix the allocator found cached: rollouts
  of one prompt compute the shared full blocks once.
* When decodes need more blocks than are free, the most recently admitted
  running sequences are preempted: their blocks are released and they go back
  to the head of the waiting queue to be prefilled again later.
* ``cache_type="none"`` keeps the reference's behaviour of recomputing the
  whole sequence every step (dense causal prefill, nothing stored).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
from torch import nn

from .attention import CacheConfig, HipPagedAttentionBackend
from .cache import CountingPagedKVCache, RadixKVCache
from .model import ModelConfig, PagedLlama, default_num_kv_blocks
from .sampling import sample_with_logprobs
from .scheduler import schedule
from .types import (EngineConfig, InferenceContext, SamplingParams, SchedulerConfig, Sequence, SequenceStatus,
                    TrainingSample)


def prefill_passes(cached: List[int], chunks: List[int]) -> List[List[int]]:
    """Row indices of a step's prefill, as one pass or two.  Two passes - rows with no cached prefix, then rows
    with one - when the rows padded to each pass's longest chunk come to at most 70 % of one batch padded to the
    longest chunk of all; the order inside a pass is the order of admission."""
    everything = list(range(len(chunks)))
    cold = [i for i in everything if cached[i] == 0]
    warm = [i for i in everything if cached[i] > 0]
    if not cold or not warm:
        return [everything]
    padded = lambda idx: len(idx) * max(chunks[i] for i in idx)
    return [cold, warm] if padded(cold) + padded(warm) <= 0.7 * padded(everything) else [everything]


class _DecodeGraph:
    """One captured forward pass of the decode step for a fixed (padded) batch size.

    Every kernel of the step reads its per-step integers (token ids, positions, slots, block tables, lengths)
    from device memory and none allocates or synchronises, so the launch sequence does not depend on their
    values: it is recorded once and replayed with the buffers rewritten in place.  Sampling stays outside."""

    def __init__(self, model: PagedLlama, batch: int, table_width: int, device: torch.device) -> None:
        self.batch, self.width = batch, table_width
        self.ids = torch.zeros((batch, 1), dtype=torch.int64, device=device)
        self.pos = torch.zeros((batch, 1), dtype=torch.int64, device=device)
        self.slots = torch.full((batch,), -1, dtype=torch.int64, device=device)
        self.tables = torch.full((batch, table_width), -1, dtype=torch.int32, device=device)
        self.lens = torch.zeros((batch,), dtype=torch.int32, device=device)
        self.ctx = InferenceContext(is_prefill=False, slot_mapping=self.slots, block_tables=self.tables,
                                    seq_lens=self.lens, max_seq_len=table_width)
        # host staging, one copy per field and step
        self._h_ids = np.zeros((batch, 1), dtype=np.int64)
        self._h_pos = np.zeros((batch, 1), dtype=np.int64)
        self._h_slots = np.full((batch,), -1, dtype=np.int64)
        self._h_tables = np.full((batch, table_width), -1, dtype=np.int32)
        self._h_lens = np.zeros((batch,), dtype=np.int32)
        # one eager pass on a side stream first (workspaces, rotary tables and library handles come into being
        # outside the capture); all rows are padding, so it writes nothing to the pool
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side), torch.no_grad():
            model(self.ids, self.pos, self.ctx)
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.hidden = model(self.ids, self.pos, self.ctx)

    def run(self, ids: np.ndarray, last_pos: np.ndarray, slots: np.ndarray, tables: np.ndarray,
            lens: np.ndarray) -> torch.Tensor:
        n = len(ids)
        if tables.shape[1] > self.width:
            raise ValueError(f"a block table of {tables.shape[1]} entries exceeds max_model_len / block_size = {self.width}")
        self._h_ids[:n] = ids
        self._h_ids[n:] = 0
        self._h_pos[:n, 0] = last_pos
        self._h_pos[n:] = 0
        self._h_slots[:n] = slots
        self._h_slots[n:] = -1
        self._h_tables.fill(-1)
        self._h_tables[:n, : tables.shape[1]] = tables
        self._h_lens[:n] = lens
        self._h_lens[n:] = 0
        for dst, src in ((self.ids, self._h_ids), (self.pos, self._h_pos), (self.slots, self._h_slots),
                         (self.tables, self._h_tables), (self.lens, self._h_lens)):
            dst.copy_(torch.from_numpy(src))
        self.graph.replay()
        return self.hidden


class InferenceEngine:
    def __init__(self, config: EngineConfig, model: Optional[PagedLlama] = None, tokenizer=None) -> None:
        assert config.block_size > 0
        assert config.max_batch_size > 0
        if config.cache_type not in ("paged", "radix", "none"):
            raise ValueError(f"unknown cache_type {config.cache_type!r}")
        self.config = config
        if not torch.cuda.is_available():
            raise RuntimeError("InferenceEngine needs a HIP device: the attention backend has no CPU implementation")
        self.device = torch.device("cuda")
        self.num_kv_blocks = config.num_kv_blocks or default_num_kv_blocks(
            config.max_batch_size, config.max_model_len, config.block_size)
        self.model = model if model is not None else self._load_model(config.model_path)
        self.backend = self.model.backend
        limit = getattr(getattr(self.model, "cfg", None), "max_position_embeddings", None)
        if limit is not None and config.max_model_len > limit:
            # the rotary tables end at max_position_embeddings; later positions would all take the last row
            raise ValueError(f"max_model_len={config.max_model_len} exceeds the model's "
                             f"max_position_embeddings={limit}")
        self.tokenizer = tokenizer if tokenizer is not None else self._load_tokenizer(config.model_path)
        self.scheduler_config = SchedulerConfig(
            max_batch_size=config.max_batch_size,
            max_tokens_per_batch=config.max_batch_size * 512,  # as the reference (engine.py:50)
            block_size=config.block_size,
        )
        self.cache = self._new_cache()
        self.waiting: List[Sequence] = []
        self.running: List[Sequence] = []
        self.seq_counter = 0
        self.weight_version = 0
        self.num_preemptions = 0
        self._decode_graphs: Dict[int, "_DecodeGraph"] = {}

    # ------------------------------------------------------------------ construction
    def _load_model(self, model_path: str) -> nn.Module:
        """A local HuggingFace checkpoint directory of the Llama / Qwen2 family (nothing is downloaded)."""
        def backend_for(cfg: ModelConfig):
            return HipPagedAttentionBackend(CacheConfig(
                num_layers=cfg.num_layers, num_kv_heads=cfg.num_kv_heads, head_dim=cfg.head_dim,
                num_blocks=self.num_kv_blocks, block_size=self.config.block_size, device="cuda",
                dtype=torch.bfloat16))
        return PagedLlama.from_local(model_path, backend_for, dtype=torch.bfloat16, device="cuda")

    @staticmethod
    def _load_tokenizer(model_path: str):
        try:
            from transformers import AutoTokenizer
            return AutoTokenizer.from_pretrained(model_path, local_files_only=True)
        except Exception:  # no tokenizer files: token-id prompts still work
            return None

    def _new_cache(self):
        if self.config.cache_type == "none":
            return None
        if self.backend.config.block_size != self.config.block_size:
            raise ValueError("EngineConfig.block_size differs from the backend's CacheConfig.block_size")
        blocks = self.backend.config.num_blocks
        cls = RadixKVCache if self.config.cache_type == "radix" else CountingPagedKVCache
        return cls(blocks, self.config.block_size)

    # ------------------------------------------------------------------ high level (engine.py:74-116)
    def generate(self, prompts: List[List[int]], sampling_params: SamplingParams,
                 num_samples_per_prompt: int = 1) -> List[TrainingSample]:
        """Completions with per-token log probabilities, ``num_samples_per_prompt`` per prompt, in the order
        in which they finish."""
        assert len(prompts) > 0
        assert num_samples_per_prompt > 0
        for prompt in prompts:
            for _ in range(num_samples_per_prompt):
                self.add_request(list(prompt), sampling_params)
        results: List[TrainingSample] = []
        while self.has_pending():
            results.extend(self.step())
        assert len(results) == len(prompts) * num_samples_per_prompt
        return results

    def generate_text(self, prompts: List[str], sampling_params: SamplingParams,
                      num_samples_per_prompt: int = 1) -> List[TrainingSample]:
        if self.tokenizer is None:
            raise RuntimeError("generate_text needs a tokenizer")
        token_prompts = [self.tokenizer.encode(p, add_special_tokens=True) for p in prompts]
        return self.generate(token_prompts, sampling_params, num_samples_per_prompt)

    # ------------------------------------------------------------------ mid level (engine.py:120-177)
    def add_request(self, prompt_tokens: List[int], params: SamplingParams) -> int:
        assert len(prompt_tokens) > 0
        if len(prompt_tokens) >= self.config.max_model_len:
            raise ValueError(f"prompt of {len(prompt_tokens)} tokens does not fit max_model_len={self.config.max_model_len}")
        seq = Sequence(
            seq_id=self.seq_counter, token_ids=list(prompt_tokens), block_ids=[],
            num_prompt_tokens=len(prompt_tokens), status=SequenceStatus.WAITING, temperature=params.temperature,
            max_tokens=params.max_tokens, stop_token_ids=params.stop_token_ids, output_logprobs=[],
        )
        self.seq_counter += 1
        self.waiting.append(seq)
        return seq.seq_id

    def step(self) -> List[TrainingSample]:
        """One scheduling decision and the forward passes it asks for; returns the sequences that finished."""
        if not self.has_pending():
            return []
        free = 1000000
        if self.cache is not None:
            # Decodes run before the prefills of the same step and take a block for every sequence whose new
            # token starts one: those blocks are not there for the prompts admitted below.
            bs = self.config.block_size
            growth = sum(1 for s in self.running[: self.scheduler_config.max_batch_size]
                         if (len(s.token_ids) - 1) % bs == 0)
            free = max(0, self.cache.num_free_blocks() - growth)
        out = schedule(self.waiting, self.running, free, self.scheduler_config)
        if self.cache is not None and not out.prefill_seqs and not out.decode_seqs and self.waiting:
            need = -(-len(self.waiting[0].token_ids) // self.config.block_size)
            raise RuntimeError(f"the KV pool ({self.backend.config.num_blocks} blocks) cannot hold a sequence of "
                               f"{need} blocks")
        decode_ids = set(out.decode_seqs)
        decode_seqs = [s for s in self.running if s.seq_id in decode_ids]
        prefill_ids = set(out.prefill_seqs)
        prefill_seqs = [s for s in self.waiting if s.seq_id in prefill_ids]
        self.waiting = [s for s in self.waiting if s.seq_id not in prefill_ids]
        for seq in prefill_seqs:
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
        finished: List[Sequence] = []
        with torch.no_grad():
            if self.cache is None:
                finished += self._recompute(prefill_seqs + decode_seqs)
            else:
                if decode_seqs:
                    finished += self._decode(self._make_room(decode_seqs))
                if prefill_seqs:
                    finished += self._prefill(prefill_seqs)
        done = {s.seq_id for s in finished}
        self.running = [s for s in self.running if s.seq_id not in done]
        return [s.to_training_sample(self.weight_version) for s in finished]

    def has_pending(self) -> bool:
        return len(self.waiting) > 0 or len(self.running) > 0

    # ------------------------------------------------------------------ weights (engine.py:183-206)
    def update_weights(self, state_dict: dict, blocking: bool = True) -> None:
        assert state_dict, "empty state_dict"
        self.model.load_state_dict(state_dict)
        self.weight_version += 1

    def get_weight_version(self) -> int:
        return self.weight_version

    def flush_cache(self) -> None:
        """Forget every cached key and value (call after a weight update).  Sequences that are running go back
        to the waiting queue and are prefilled again under the new weights."""
        for seq in reversed(self.running):
            seq.status = SequenceStatus.WAITING
            seq.block_ids = []
            self.waiting.insert(0, seq)
        self.running = []
        self.backend.clear_cache()
        self.cache = self._new_cache()

    def shutdown(self) -> None:
        self._decode_graphs.clear()
        self.waiting.clear()
        self.running.clear()
        self.cache = self._new_cache()

    # ------------------------------------------------------------------ forward passes
    def _make_room(self, decode_seqs: List[Sequence]) -> List[Sequence]:
        """Preempt from the most recently admitted end until the decodes that start a new block fit."""
        bs = self.config.block_size
        keep = list(decode_seqs)
        while keep:
            need = sum(1 for s in keep if (len(s.token_ids) - 1) % bs == 0)
            if need <= self.cache.num_free_blocks():
                break
            self._preempt(keep.pop())
        return keep

    def _defer(self, seqs: List[Sequence]) -> None:
        """Sequences admitted for prefill whose blocks could not be had: back to the head of the waiting queue,
        in their order, untouched."""
        ids = {s.seq_id for s in seqs}
        self.running = [s for s in self.running if s.seq_id not in ids]
        for s in reversed(seqs):
            s.status = SequenceStatus.WAITING
            s.block_ids = []
            self.waiting.insert(0, s)

    def _preempt(self, seq: Sequence) -> None:
        self.cache.deallocate(seq.seq_id)
        seq.status = SequenceStatus.WAITING
        seq.block_ids = []
        self.running = [s for s in self.running if s.seq_id != seq.seq_id]
        self.waiting.insert(0, seq)
        self.num_preemptions += 1

    def _tables(self, seqs: List[Sequence]) -> np.ndarray:
        width = max(len(s.block_ids) for s in seqs)
        tables = np.full((len(seqs), width), -1, dtype=np.int32)
        for i, s in enumerate(seqs):
            tables[i, : len(s.block_ids)] = s.block_ids
        return tables

    def _prefill(self, seqs: List[Sequence]) -> List[Sequence]:
        cached, chunks = [], []
        for i, s in enumerate(seqs):
            try:
                s.block_ids = list(self.cache.allocate(s.seq_id, s.token_ids))
            except RuntimeError:
                # The pool ran short after all (the schedule counts free blocks, not which of them hold a
                # prefix this prompt will revive): this prompt and the ones admitted after it wait a step.
                self._defer(seqs[i:])
                seqs = seqs[:i]
                break
            n = len(s.token_ids)
            c = min(self.cache.get_cached_tokens(s.seq_id), n - 1)  # the last token is always computed: its
            cached.append(c)                                         # hidden state gives the next token
            chunks.append(n - c)
        # One batched forward pads every row to the longest chunk.  N rollouts of one prompt arrive as one row
        # with the whole prompt and N-1 rows with a single uncached token, so the rows are split in two passes
        # when that removes most of the padding: first the rows with no cached prefix (they depend on nothing
        # and write the blocks that later rows share), then the rows with one (their prefix blocks were written
        # in an earlier step, by the first pass, or by an earlier row of their own pass, whose append precedes
        # the attention inside every layer).
        finished: List[Sequence] = []
        if not seqs:
            return finished
        for idx in prefill_passes(cached, chunks):
            finished += self._prefill_rows([seqs[i] for i in idx], [cached[i] for i in idx],
                                           [chunks[i] for i in idx])
        return finished

    def _prefill_rows(self, seqs: List[Sequence], cached: List[int], chunks: List[int]) -> List[Sequence]:
        bs = self.config.block_size
        t_max = max(chunks)
        ids = np.zeros((len(seqs), t_max), dtype=np.int64)
        pos = np.zeros((len(seqs), t_max), dtype=np.int64)
        slots = np.full((len(seqs), t_max), -1, dtype=np.int64)
        for i, s in enumerate(seqs):
            p = np.arange(cached[i], len(s.token_ids))
            ids[i, : chunks[i]] = s.token_ids[cached[i]:]
            pos[i, : chunks[i]] = p
            slots[i, : chunks[i]] = np.asarray(s.block_ids, dtype=np.int64)[p // bs] * bs + p % bs
        totals = np.asarray([len(s.token_ids) for s in seqs], dtype=np.int64)
        ctx = InferenceContext(is_prefill=True, slot_mapping=slots.reshape(-1), block_tables=self._tables(seqs),
                               seq_lens=totals, max_seq_len=int(totals.max()),
                               prefix_lens=np.asarray(cached, dtype=np.int64))
        hidden = self.model(torch.from_numpy(ids).to(self.device), torch.from_numpy(pos).to(self.device), ctx)
        last = hidden[torch.arange(len(seqs), device=self.device),
                      torch.tensor([c - 1 for c in chunks], device=self.device)]
        return self._sample(seqs, last)

    def _decode(self, seqs: List[Sequence]) -> List[Sequence]:
        if not seqs:
            return []
        for s in seqs:
            self.cache.append_token(s.seq_id, s.token_ids[-1])  # hands out a block when the token starts one
            s.block_ids = list(self.cache.get_block_ids(s.seq_id))
        return self._decode_rows(seqs)

    def _decode_rows(self, seqs: List[Sequence]) -> List[Sequence]:
        bs = self.config.block_size
        lens = np.asarray([len(s.token_ids) for s in seqs], dtype=np.int64)
        last_pos = lens - 1
        ids = np.asarray([[s.token_ids[-1]] for s in seqs], dtype=np.int64)
        slots = np.asarray([s.block_ids[p // bs] * bs + p % bs for s, p in zip(seqs, last_pos)], dtype=np.int64)
        ctx = InferenceContext(is_prefill=False, slot_mapping=slots, block_tables=self._tables(seqs), seq_lens=lens,
                               max_seq_len=int(lens.max()))
        if self.config.use_graphs:
            hidden = self._decode_replay(ids, last_pos, slots, ctx.block_tables, lens)
        else:
            hidden = self.model(torch.from_numpy(ids).to(self.device),
                                torch.from_numpy(last_pos[:, None].copy()).to(self.device), ctx)
        return self._sample(seqs, hidden[:, 0])

    def _decode_replay(self, ids: np.ndarray, last_pos: np.ndarray, slots: np.ndarray, tables: np.ndarray,
                       lens: np.ndarray) -> torch.Tensor:
        """The decode step's forward pass from a captured graph.  Batches are padded to a bucket size with
        sequences of length 0 and slot -1 (nothing is written, their rows are ignored); the graph reads token
        ids, positions, slots, block tables and lengths from buffers that are rewritten before every replay."""
        n = len(ids)
        bucket = 8
        while bucket < n:
            bucket *= 2
        bucket = min(bucket, max(self.config.max_batch_size, n))
        g = self._decode_graphs.get(bucket)
        if g is None:
            width = -(-self.config.max_model_len // self.config.block_size)
            g = self._decode_graphs[bucket] = _DecodeGraph(self.model, bucket, width, self.device)
        return g.run(ids, last_pos, slots, tables, lens)[:n]

    def _recompute(self, seqs: List[Sequence]) -> List[Sequence]:
        """The reference's cache-less step: every sequence's whole token list, one at a time (engine.py:218-250)."""
        finished: List[Sequence] = []
        for s in seqs:
            ids = torch.tensor([s.token_ids], device=self.device)
            pos = torch.arange(len(s.token_ids), device=self.device)[None]
            hidden = self.model(ids, pos, InferenceContext(is_prefill=True))
            finished += self._sample([s], hidden[:, -1])
        return finished

    def _sample(self, seqs: List[Sequence], last_hidden: torch.Tensor) -> List[Sequence]:
        logits = self.model.logits(last_hidden).float()
        temps = torch.tensor([s.temperature for s in seqs], device=self.device, dtype=torch.float32)
        tokens, logprobs = sample_with_logprobs(logits, temps)
        tokens, logprobs = tokens.tolist(), logprobs.tolist()
        finished: List[Sequence] = []
        for seq, token, logprob in zip(seqs, tokens, logprobs):
            seq.append_token(token, logprob)
            if self._should_stop(seq, token):
                seq.status = SequenceStatus.FINISHED
                if self.cache is not None:
                    self.cache.deallocate(seq.seq_id)
                finished.append(seq)
        return finished

    def _should_stop(self, seq: Sequence, token_id: int) -> bool:
        if token_id in seq.stop_token_ids:
            return True
        eos = self.tokenizer.eos_token_id if self.tokenizer is not None else self.config.eos_token_id
        if eos is not None and token_id == eos:
            return True
        return seq.num_generated >= seq.max_tokens or len(seq.token_ids) >= self.config.max_model_len
