"""Continuous-batching scheduler (iteration-level, prefill-first), microbatch aware.

Replaces the reference's one-request-at-a-time worker (1 sync gunicorn worker,
``worker/Dockerfile:45``; batch = 1): every engine step either admits a packed batch of
waiting prompts (prefill) or advances every running sequence of one microbatch by one
token (decode). With pipeline parallelism the running set is split into M microbatches
(M = number of stages) that circulate through the pipeline; each microbatch is scheduled
only after its previous step's tokens came back.

The decode path is vectorised: each microbatch keeps numpy state (ids, context lengths,
token budgets, sampling params) rebuilt only when its membership changes, and the C++
``BlockManager`` builds slot mappings / block tables for the whole batch in one call, so
scheduling 256 sequences costs ~0.1 ms of host time (it gates every pipeline tick).

KV memory comes from the C++ allocator; when a decode step cannot get a block the newest
sequence of that microbatch is preempted (blocks freed, re-queued at the front, recomputed
later from prompt + generated tokens).
"""
from __future__ import annotations

import itertools
import os
import time
import zlib
from collections import deque
from typing import Dict, List, Optional

import numpy as np

from ..runtime import BlockManager
from .batch import DECODE, PREFILL, StepMeta
from .sequence import SamplingParams, Sequence, SeqState, row_seed

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def row_seeds(seq_seeds: np.ndarray, index: np.ndarray) -> np.ndarray:
    """Vectorised ``sequence.row_seed`` (splitmix64 of (seed, output index))."""
    with np.errstate(over="ignore"):
        z = (seq_seeds.astype(np.uint64) * np.uint64(0x9E3779B97F4A7C15)
             + index.astype(np.uint64) + np.uint64(0x632BE59BD9B4E019))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z.view(np.int64)


class _MBState:
    """numpy mirror of one microbatch's running sequences (decode fast path).

    Tokens generated since the mirror was built are kept in ``hist`` (one column per step,
    every row advances together on the fast path) and appended to the sequences'
    ``output_ids`` only when a row leaves (finish / preemption) or the mirror is dropped
    (``flush``): no per-token Python work per step. Finished rows are removed by
    ``compact`` instead of rebuilding the mirror."""
    __slots__ = ("seqs", "sid", "ctx", "out_cnt", "budget", "last", "temp", "topk", "topp",
                 "seed", "eos_ok", "stops", "first_pending", "hist", "k")

    def __init__(self, seqs: List[Sequence], eos: Optional[int]):
        self.seqs = list(seqs)
        n = len(seqs)
        self.sid = np.fromiter((s.seq_id for s in seqs), np.int64, n)
        self.ctx = np.fromiter((s.total_len for s in seqs), np.int32, n)
        self.out_cnt = np.fromiter((len(s.output_ids) for s in seqs), np.int32, n)
        self.budget = np.fromiter((s.params.budget(s.prompt_len) for s in seqs), np.int32, n)
        self.last = np.fromiter(((s.output_ids[-1] if s.output_ids else s.prompt_ids[-1])
                                 for s in seqs), np.int32, n)
        self.temp = np.fromiter((s.params.effective_temperature() for s in seqs), np.float32, n)
        self.topk = np.fromiter((s.params.top_k for s in seqs), np.int32, n)
        self.topp = np.fromiter((s.params.top_p for s in seqs), np.float32, n)
        self.seed = np.fromiter((s.seed for s in seqs), np.int64, n)
        self.eos_ok = np.fromiter((eos is not None and not s.params.ignore_eos for s in seqs),
                                  bool, n)
        self.stops = [i for i, s in enumerate(seqs) if s.params.stop_token_ids]
        self.first_pending = bool((self.out_cnt == 0).any())
        left = int((self.budget - self.out_cnt).max()) if n else 0
        self.hist = np.zeros((n, max(1, min(left, 4096))), dtype=np.int32)
        self.k = 0

    def record(self, tokens: np.ndarray) -> None:
        if self.k >= self.hist.shape[1]:
            self.hist = np.concatenate([self.hist, np.zeros_like(self.hist)], axis=1)
        self.hist[:, self.k] = tokens
        self.k += 1

    def flush_rows(self, idx) -> None:
        """Append the pending tokens of rows ``idx`` to their sequences."""
        if self.k == 0:
            return
        for i in idx:
            self.seqs[i].output_ids.extend(self.hist[i, :self.k].tolist())

    def flush(self) -> None:
        self.flush_rows(range(len(self.seqs)))
        self.hist[:, :self.k] = 0
        self.k = 0

    def compact(self, keep: np.ndarray) -> None:
        """Drop rows where ``keep`` is False (their tokens must have been flushed)."""
        for name in ("sid", "ctx", "out_cnt", "budget", "last", "temp", "topk", "topp", "seed",
                     "eos_ok", "hist"):
            setattr(self, name, getattr(self, name)[keep])
        new_idx = np.cumsum(keep) - 1
        self.stops = [int(new_idx[i]) for i in self.stops if keep[i]]
        self.seqs = [s for s, kp in zip(self.seqs, keep.tolist()) if kp]


class _MBCore:
    """The same mirror in C++ (``runtime.DecodeCore``): the decode fast path of the pipeline
    head, where one tick's scheduling + token application must cost tens of microseconds.
    Used when no lookahead is involved and no row has stop tokens."""
    __slots__ = ("seqs", "core", "first_rows", "vp")

    def __init__(self, seqs: List[Sequence], eos: Optional[int], max_model_len: int):
        from ..runtime import DecodeCore
        self.seqs = list(seqs)
        self.vp = None           # (rows, flag): pipeline head's vocab-parallel check, cached
        n = len(seqs)
        out_cnt = np.fromiter((len(s.output_ids) for s in seqs), np.int32, n)
        budget = np.fromiter((s.params.budget(s.prompt_len) for s in seqs), np.int32, n)
        self.first_rows = np.nonzero(out_cnt == 0)[0].tolist()
        left = int((budget - out_cnt).max()) if n else 1
        self.core = DecodeCore(
            np.fromiter((s.seq_id for s in seqs), np.int64, n),
            np.fromiter((s.total_len for s in seqs), np.int32, n), out_cnt, budget,
            np.fromiter(((s.output_ids[-1] if s.output_ids else s.prompt_ids[-1])
                         for s in seqs), np.int32, n),
            np.fromiter((s.params.effective_temperature() for s in seqs), np.float32, n),
            np.fromiter((s.params.top_k for s in seqs), np.int32, n),
            np.fromiter((s.params.top_p for s in seqs), np.float32, n),
            np.fromiter((s.seed for s in seqs), np.int64, n),
            np.fromiter((eos is not None and not s.params.ignore_eos for s in seqs), bool, n),
            eos, max_model_len, max(1, min(left, 4096)))

    def flush(self) -> None:
        h = self.core.history()
        if h.shape[1]:
            for s, row in zip(self.seqs, h.tolist()):
                s.output_ids.extend(row)


try:                                   # 64-bit block hashes (collisions ~2^-64 per pair)
    import xxhash as _xxhash

    def _hash64(b: bytes) -> int:
        return _xxhash.xxh3_64_intdigest(b)
except ImportError:                    # pragma: no cover - xxhash ships in the image
    import hashlib as _hashlib

    def _hash64(b: bytes) -> int:
        return int.from_bytes(_hashlib.blake2b(b, digest_size=8).digest(), "little")


class Scheduler:
    def __init__(self, block_manager: BlockManager, max_seqs_per_mb: int = 256,
                 max_prefill_tokens: int = 16384, num_microbatches: int = 1,
                 eos_token_id: Optional[int] = None, max_model_len: int = 4096,
                 table_width: Optional[int] = None, native_decode: bool = False,
                 admit_window_s: Optional[float] = None, admit_min_frac: float = 0.125,
                 refill_interval_s: Optional[float] = None,
                 prefix_caching: Optional[bool] = None, mixed_steps: bool = False,
                 state_slots=None, always_paged: bool = False):
        self.bm = block_manager
        # models with a recurrent state per sequence: a slot per admitted sequence
        # (engine.kv_cache.StateSlots), released with the sequence's blocks
        self.state_slots = state_slots
        # models that attend through the paged cache in every step kind get block tables
        # (and context lengths) on whole-prompt prefill steps too
        self.always_paged = bool(always_paged)
        self._replay: Dict[str, Sequence] = {}
        self.bs = block_manager.block_size
        self.max_seqs = max_seqs_per_mb
        self.max_prefill_tokens = max_prefill_tokens
        self.M = num_microbatches
        self.eos = eos_token_id
        self.max_model_len = max_model_len
        # fixed block-table width (static for hipGraph replay) = blocks for max_model_len
        self.table_width = table_width or -(-max_model_len // self.bs)
        self.waiting: deque = deque()
        self.running: List[List[Sequence]] = [[] for _ in range(self.M)]
        # chunked prefill: prompts longer than max_prefill_tokens are prefilled over several
        # steps (their KV blocks are held from the first chunk on); between two chunk steps of
        # a microbatch that is also decoding, one decode step runs, so a long prompt delays
        # the running sequences' next token by at most one chunk
        self.prefilling: List[List[Sequence]] = [[] for _ in range(self.M)]
        self._chunk_turn = [True] * self.M
        self._state: List[Optional[_MBState]] = [None] * self.M
        self.seqs: Dict[int, Sequence] = {}
        self.finished: List[Sequence] = []
        # decode fast path in C++ (runtime.DecodeCore) for microbatches without stop tokens
        self.native_decode = native_decode
        # admission window: while a microbatch is decoding, a prefill step for it waits until
        # max(1, admit_min_frac * max_seqs) requests are queued (or as many as fit) or the
        # oldest has waited admit_window_s. A prefill streams every weight like a decode step
        # does, so admitting requests one by one as they trickle in over HTTP halves decode
        # throughput; the window bounds the added time-to-first-token instead.
        self.admit_window_s = (float(os.environ.get("DLI_ADMIT_WINDOW_S", "0.02"))
                               if admit_window_s is None else admit_window_s)
        self.admit_min = max(1, int(admit_min_frac * max_seqs_per_mb))
        # refill pacing: while a microbatch is nearly full (fewer than admit_min free slots)
        # and requests keep queueing (more in flight than slots), every decode step frees a
        # few slots; refilling them at once runs a prefill step per decode step (measured end
        # to end at concurrency 1024: 503 prefill steps of ~8 prompts for 646 decode steps).
        # Such refills wait until admit_min slots are free or refill_interval_s has passed
        # since the microbatch's last admission.
        self.refill_interval_s = (float(os.environ.get("DLI_REFILL_INTERVAL_S", "0.06"))
                                  if refill_interval_s is None else refill_interval_s)
        self._last_admit = [0.0] * num_microbatches
        # automatic prefix caching: a new sequence maps the cached KV blocks of its longest
        # known full-block prefix (chain hashes of the token blocks) and prefills only the
        # rest, as a chunk over the paged cache; full prompt blocks are published when their
        # prefill is scheduled (the device runs steps in order)
        self.prefix_caching = (os.environ.get("DLI_PREFIX_CACHE", "1") == "1"
                               if prefix_caching is None else bool(prefix_caching))
        self.prefix_hit_tokens = 0
        # mixed steps: a prefill step of a microbatch that is also decoding carries the running
        # sequences' decode rows too (one token each, ahead of the prompt rows), so admitting
        # prompts or prefilling a chunk no longer stalls the running sequences for a step and
        # their rows ride on the prefill's (compute-bound) GEMMs instead of costing a separate
        # weight-streaming decode step. Pipelines use them too: the decode-row count crosses
        # the stages in header word 9 of the packed step metadata (StepMeta.pack).
        self.mixed_steps = bool(mixed_steps)
        self.num_mixed = 0
        self.num_preempted = 0
        self._next_id = 0
        self._step = 0
        self._deadlines = 0

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id: str, prompt_ids: List[int],
                    params: Optional[SamplingParams] = None) -> Sequence:
        params = params or SamplingParams()
        if len(prompt_ids) == 0:
            raise ValueError("empty prompt")
        if len(prompt_ids) >= self.max_model_len:
            raise ValueError(f"prompt of {len(prompt_ids)} tokens exceeds max_model_len "
                             f"{self.max_model_len}")
        sid = self._next_id
        self._next_id += 1
        seed = (params.seed if params.seed is not None
                else zlib.crc32(f"{request_id}:{sid}".encode()) & 0x7FFFFFFF)
        seq = Sequence(seq_id=sid, request_id=request_id, prompt_ids=list(prompt_ids),
                       params=params, seed=int(seed))
        self.seqs[sid] = seq
        if params.timeout_s is not None:
            self._deadlines += 1
        if params.budget(len(prompt_ids)) <= 0:
            self._finish(seq, "length")
        else:
            self.waiting.append(seq)
        return seq

    def abort(self, request_id: str) -> bool:
        for seq in list(self.seqs.values()):
            if seq.request_id == request_id and seq.state != SeqState.FINISHED:
                self._finish(seq, "abort")
                return True
        return False

    def has_work(self) -> bool:
        return bool(self.waiting) or any(self.running) or any(self.prefilling)

    def num_running(self) -> int:
        return sum(len(r) for r in self.running)

    # ------------------------------------------------------------------ internals
    def _drop_state(self, mb: int) -> None:
        st = self._state[mb]
        if st is not None:
            st.flush()
            self._state[mb] = None

    def _finish(self, seq: Sequence, reason: str):
        if seq.state == SeqState.FINISHED:
            return
        if seq.state == SeqState.WAITING:
            try:
                self.waiting.remove(seq)
            except ValueError:
                pass
        elif seq.state == SeqState.RUNNING:
            self._drop_state(seq.microbatch)
            r = self.running[seq.microbatch]
            try:
                r.remove(seq)
            except ValueError:
                pass
        elif seq.state == SeqState.PREFILLING:
            try:
                self.prefilling[seq.microbatch].remove(seq)
            except ValueError:
                pass
        self._mark_finished(seq, reason)

    def _mark_finished(self, seq: Sequence, reason: str, free: bool = True):
        seq.state = SeqState.FINISHED
        seq.finish_reason = reason
        seq.finish_time = time.perf_counter()
        if free:
            self.bm.free(seq.seq_id)
        if self.state_slots is not None:
            self.state_slots.release(seq.seq_id)
        if seq.params.timeout_s is not None:
            self._deadlines -= 1
        self.finished.append(seq)

    def _expire(self):
        if self._deadlines <= 0:
            return
        now = time.perf_counter()
        for seq in (list(self.waiting) + [s for r in self.running for s in r] +
                    [s for r in self.prefilling for s in r]):
            dl = seq.deadline
            if dl is not None and now > dl:
                self._finish(seq, "timeout")

    def _preempt(self, mb: int) -> bool:
        r = self.running[mb]
        if not r:
            return False
        self._drop_state(mb)
        victim = max(r, key=lambda s: s.arrival)
        r.remove(victim)
        self.bm.free(victim.seq_id)
        if self.state_slots is not None:
            self.state_slots.release(victim.seq_id)
        victim.state = SeqState.WAITING
        victim.num_prefilled = 0
        victim.num_preemptions += 1
        victim.preempt_step = self._step
        self.num_preempted += 1
        self.waiting.appendleft(victim)
        return True

    def _slots_of(self, seqs) -> Optional[np.ndarray]:
        """State slot of each sequence (acquired at its first step), None without slots."""
        if self.state_slots is None:
            return None
        out = np.fromiter((self.state_slots.acquire(s.seq_id) for s in seqs), np.int32,
                          len(seqs))
        if (out < 0).any():
            raise RuntimeError("no free recurrent-state slot (more live sequences than slots)")
        return out

    def _sampling_arrays(self, seqs: List[Sequence]):
        n = len(seqs)
        temp = np.fromiter((s.params.effective_temperature() for s in seqs), np.float32, n)
        topk = np.fromiter((s.params.top_k for s in seqs), np.int32, n)
        topp = np.fromiter((s.params.top_p for s in seqs), np.float32, n)
        seeds = row_seeds(np.fromiter((s.seed for s in seqs), np.int64, n),
                          np.fromiter((len(s.output_ids) for s in seqs), np.int64, n))
        return temp, topk, topp, seeds

    # ------------------------------------------------------------------ scheduling
    def schedule(self, mb: int = 0, inflight: Optional[StepMeta] = None) -> Optional[StepMeta]:
        """Next step for microbatch ``mb`` (None if it has nothing to do).

        ``inflight``: a step of this microbatch whose tokens have not been applied yet
        (lookahead scheduling, one step ahead of the host). Its sequences are scheduled as if
        each had produced one more non-stop token: context and output index advance by one,
        those that reach their length budget with it are left out, and their input id comes
        from the in-flight step's device output (``meta.feed_src`` = row in that output, -1 =
        host id). A sequence that instead stops on EOS wastes one row of the next step; its
        token is dropped by ``update`` (the sequence is no longer running)."""
        self._expire()
        self._step += 1
        if self.mixed_steps and self.running[mb] and (self.waiting or self.prefilling[mb]):
            # the decode rows are scheduled first, against the sequences running before this
            # step's admissions (a prompt finishing its prefill here has no token to feed yet)
            npre = self.num_preempted
            dec = self._decode(mb, inflight, allow_native=False)
            # a sequence the decode half just preempted may still be in the in-flight step:
            # it is not re-admitted by this step's prefill half (it waits one step)
            pre = self._try_prefill(mb, mixed=True) if self.num_preempted == npre else None
            if pre is None or dec is None:
                return dec if pre is None else pre
            return self._merge(dec, pre)
        meta = self._try_prefill(mb)
        if meta is not None:
            return meta
        return self._decode(mb, inflight)

    def _merge(self, dec: StepMeta, pre: StepMeta) -> StepMeta:
        """One PREFILL-kind step: ``dec``'s decode rows (one token each) then ``pre``'s prompt
        chunks. Its tokens are applied by the per-sequence update path (the microbatch's
        decode state is dropped), rows of unfinished chunks masked out."""
        mb = dec.microbatch
        self._drop_state(mb)
        nd, npf = dec.num_seqs, pre.num_seqs
        width = max(dec.block_tables.shape[1], pre.block_tables.shape[1])

        def pad(t):
            return t if t.shape[1] == width else np.pad(t, ((0, 0), (0, width - t.shape[1])))
        sid = np.concatenate([np.asarray(dec.seq_ids_arr if dec.seq_ids_arr is not None
                                         else dec.seq_ids, np.int64), pre.seq_ids_arr])
        cat = np.concatenate
        meta = StepMeta(kind=PREFILL, seq_ids=sid.tolist(),
                        input_ids=cat([np.asarray(dec.input_ids, np.int32), pre.input_ids]),
                        positions=cat([np.asarray(dec.positions, np.int32), pre.positions]),
                        slot_mapping=cat([np.asarray(dec.slot_mapping, np.int32),
                                          pre.slot_mapping]),
                        seq_lens=cat([np.ones(nd, np.int32), pre.seq_lens]),
                        context_lens=cat([np.asarray(dec.context_lens, np.int32),
                                          pre.context_lens]),
                        block_tables=cat([pad(np.asarray(dec.block_tables, np.int32)),
                                          pad(np.asarray(pre.block_tables, np.int32))]),
                        temperature=cat([dec.temperature, pre.temperature]),
                        top_k=cat([dec.top_k, pre.top_k]), top_p=cat([dec.top_p, pre.top_p]),
                        seeds=cat([dec.seeds, pre.seeds]), microbatch=mb, step_id=pre.step_id,
                        seq_ids_arr=sid)
        meta.num_decode = nd
        if dec.state_slots is not None:
            meta.state_slots = cat([dec.state_slots, pre.state_slots])
        if dec.feed_src is not None:
            meta.feed_src = cat([dec.feed_src, np.full(int(pre.num_tokens), -1, np.int32)])
        if pre.sample_mask is not None:
            meta.sample_mask = cat([np.ones(nd, np.bool_), pre.sample_mask])
        self.num_mixed += 1
        return meta

    def _least_loaded_ok(self, mb: int) -> bool:
        # balance admissions across microbatches: only admit into mb if it is among the least loaded
        loads = [len(r) for r in self.running]
        return len(self.running[mb]) <= min(loads)

    def _block_hashes(self, seq: Sequence, nblocks: int) -> np.ndarray:
        """Chain hashes of the first ``nblocks`` full token blocks of ``seq`` (a block's hash
        covers every token before it too)."""
        ids = np.asarray(seq.prompt_ids + seq.output_ids if seq.output_ids else seq.prompt_ids,
                         dtype=np.int32)
        bs = self.bs
        out = np.empty(nblocks, np.uint64)
        h = 0
        for i in range(nblocks):
            h = _hash64(h.to_bytes(8, "little") + ids[i * bs:(i + 1) * bs].tobytes()) or 1
            out[i] = h
        return out

    def _match_prefix(self, seq: Sequence) -> None:
        if not self.prefix_caching or seq.num_prefilled or seq.total_len <= self.bs:
            return
        nb = (seq.total_len - 1) // self.bs          # keep >= 1 token to compute
        m = self.bm.match_prefix(seq.seq_id, self._block_hashes(seq, nb))
        if m:
            seq.num_prefilled = m * self.bs
            self.prefix_hit_tokens += m * self.bs

    def _unmatch(self, seq: Sequence) -> None:
        if seq.num_prefilled:
            self.bm.free(seq.seq_id)
            self.prefix_hit_tokens -= seq.num_prefilled
            seq.num_prefilled = 0

    def _try_prefill(self, mb: int, mixed: bool = False) -> Optional[StepMeta]:
        """``mixed``: the step also carries the microbatch's decode rows (chunks then run every
        step, and the block tables are always built: the mixed step attends over the cache)."""
        partial = self.prefilling[mb]
        if partial and not mixed:
            # a chunk step every other step while the microbatch also decodes
            if self.running[mb] and not self._chunk_turn[mb]:
                self._chunk_turn[mb] = True
                return None
            self._chunk_turn[mb] = False
        if not partial:
            if not self.waiting or (self.M > 1 and not self._least_loaded_ok(mb)):
                return None
            if self.running[mb] and self.admit_window_s > 0:
                now = time.perf_counter()
                free = self.max_seqs - len(self.running[mb])
                want = min(self.admit_min, free)
                if (len(self.waiting) < want and
                        now - self.waiting[0].arrival < self.admit_window_s):
                    return None              # keep decoding; batch the arrivals
                if (free < self.admit_min and self.refill_interval_s > 0
                        and now - self._last_admit[mb] < self.refill_interval_s):
                    return None              # nearly full: pace the refills
        budget = self.max_prefill_tokens
        picked: List[Sequence] = []
        starts_l: List[int] = []
        lens_l: List[int] = []
        for seq in partial:                  # continue chunked prompts first, in order
            if budget <= 0:
                break
            n = min(seq.total_len - seq.num_prefilled, budget)
            picked.append(seq)
            starts_l.append(seq.num_prefilled)
            lens_l.append(n)
            budget -= n
        n_cont = len(picked)
        new: List[Sequence] = []
        new_lens: List[int] = []
        room = self.max_seqs - len(self.running[mb]) - len(partial)
        if budget > 0 and room > 0 and not (self.M > 1 and n_cont == 0
                                            and not self._least_loaded_ok(mb)):
            for seq in self.waiting:
                if len(new) >= room or budget <= 0:
                    break
                self._match_prefix(seq)              # cached prefix blocks need no prefill
                n = seq.total_len - seq.num_prefilled
                if n > budget and (new or n_cont or n <= self.max_prefill_tokens):
                    self._unmatch(seq)
                    break                    # whole prompts only, except a chunked first
                new.append(seq)
                new_lens.append(seq.total_len)
                budget -= min(n, budget)
        if new:
            self._last_admit[mb] = time.perf_counter()
            # blocks for every new prompt (whole length, also when chunked) in one C++ call;
            # stops at the first that does not fit
            sid_new = np.fromiter((s.seq_id for s in new), np.int64, len(new))
            got = self.bm.ensure_batch(sid_new, np.asarray(new_lens, dtype=np.int32))
            for s in new[got:]:
                self._unmatch(s)
            new = new[:got]
            for _ in range(got):
                self.waiting.popleft()
            budget = self.max_prefill_tokens - sum(lens_l)
            for s in new:
                n = min(s.total_len - s.num_prefilled, budget)
                picked.append(s)
                starts_l.append(s.num_prefilled)
                lens_l.append(n)
                budget -= n
        if not picked:
            return None
        S = len(picked)
        sid = np.fromiter((s.seq_id for s in picked), np.int64, S)
        starts = np.asarray(starts_l, dtype=np.int32)
        lens = np.asarray(lens_l, dtype=np.int32)
        chunked = any(st > 0 or st + n < s.total_len
                      for s, st, n in zip(picked, starts_l, lens_l))
        final = np.fromiter((st + n == s.total_len for s, st, n in zip(picked, starts_l, lens_l)),
                            np.bool_, S)
        joined = False
        for s, st, n, f in zip(picked, starts_l, lens_l, final.tolist()):
            s.num_prefilled = st + n
            s.microbatch = mb
            if f:
                if s.state == SeqState.PREFILLING:
                    partial.remove(s)
                s.state = SeqState.RUNNING
                self.running[mb].append(s)
                joined = True
                if self.prefix_caching and s.total_len >= self.bs:
                    self.bm.register_prefix(s.seq_id,
                                            self._block_hashes(s, s.total_len // self.bs))
            elif s.state != SeqState.PREFILLING:
                s.state = SeqState.PREFILLING
                partial.append(s)
        if joined:
            self._drop_state(mb)
        T = int(lens.sum())
        if chunked:
            ids = np.fromiter(itertools.chain.from_iterable(
                (s.prompt_ids + s.output_ids)[st:st + n]
                for s, st, n in zip(picked, starts_l, lens_l)), np.int32, T)
        else:
            ids = np.fromiter(itertools.chain.from_iterable(
                (s.prompt_ids + s.output_ids) if s.output_ids else s.prompt_ids for s in picked),
                np.int32, T)
        cu = np.zeros(S, np.int32)
        cu[1:] = np.cumsum(lens)[:-1]
        pos = (np.arange(T, dtype=np.int32) - np.repeat(cu - starts, lens)).astype(np.int32)
        slots = self.bm.slot_mapping(sid, starts, lens)
        ctx = starts + lens
        if chunked or mixed or self.always_paged:
            width = -(-max(s.total_len for s in picked) // self.bs)   # blocks held per seq
            tables = self.bm.fill_tables(sid.tolist(), width)
        else:
            tables = np.zeros((S, 0), np.int32)
        temp, topk, topp, seeds = self._sampling_arrays(picked)
        meta = StepMeta(kind=PREFILL, seq_ids=sid.tolist(), input_ids=ids, positions=pos,
                        slot_mapping=slots, seq_lens=lens, context_lens=ctx,
                        block_tables=tables, temperature=temp, top_k=topk, top_p=topp,
                        seeds=seeds, microbatch=mb, step_id=self._step, seq_ids_arr=sid)
        if not final.all():
            meta.sample_mask = final
        meta.state_slots = self._slots_of(picked)
        return meta

    def _mb_state(self, mb: int, native: bool = False):
        st = self._state[mb]
        if st is not None and native != isinstance(st, _MBCore):
            self._drop_state(mb)
            st = None
        if st is None:
            if native:
                st = _MBCore(self.running[mb], self.eos, self.max_model_len)
            else:
                st = _MBState(self.running[mb], self.eos)
            self._state[mb] = st
        return st

    @staticmethod
    def _advance(st: _MBState, inflight: Optional[StepMeta]):
        """(adv, src): adv[i] = 1 if sequence i is in the in-flight step (its token is not
        applied yet), src[i] = its row in that step's output (-1 otherwise)."""
        n = len(st.seqs)
        if inflight is None or inflight.num_seqs == 0:
            return np.zeros(n, np.int32), np.full(n, -1, np.int32)
        ks = np.asarray(inflight.seq_ids, dtype=np.int64)
        order = np.argsort(ks, kind="stable")
        sk = ks[order]
        pos = np.minimum(np.searchsorted(sk, st.sid), len(sk) - 1)
        hit = sk[pos] == st.sid
        return hit.astype(np.int32), np.where(hit, order[pos], -1).astype(np.int32)

    def _native_ok(self, mb: int, inflight: Optional[StepMeta]) -> bool:
        if not self.native_decode or inflight is not None:
            return False
        st = self._state[mb]
        if isinstance(st, _MBCore):
            return True
        return not any(s.params.stop_token_ids for s in self.running[mb])

    def _decode_native(self, mb: int) -> Optional[StepMeta]:
        while True:
            st = self._mb_state(mb, native=True)
            S = len(st.seqs)
            if S == 0:
                return None
            payload, cols = st.core.schedule(self.bm, self.table_width)
            if payload is not None:
                break
            if not self._preempt(mb):
                return None
        o = [0]

        def take(n, dt=None):
            v = payload[o[0]:o[0] + n]
            o[0] += n
            return v if dt is None else v.view(dt)
        sid = take(S)
        ids, pos, slots, lens, ctx = take(S), take(S), take(S), take(S), take(S)
        tables = take(S * cols).reshape(S, cols)
        temp, topk, topp = take(S, np.float32), take(S), take(S, np.float32)
        seeds = take(2 * S, np.int64)
        meta = StepMeta(kind=DECODE, seq_ids=sid, input_ids=ids, positions=pos,
                        slot_mapping=slots, seq_lens=lens, context_lens=ctx, block_tables=tables,
                        temperature=temp, top_k=topk, top_p=topp, seeds=seeds, microbatch=mb,
                        step_id=self._step)
        meta.table_used = cols
        meta.packed_payload = payload
        meta.table_width_full = self.table_width
        meta.core = (st, st.core.steps, S)
        return meta

    def _decode(self, mb: int, inflight: Optional[StepMeta] = None,
                allow_native: bool = True) -> Optional[StepMeta]:
        if not self.running[mb]:
            return None
        if allow_native and self._native_ok(mb, inflight):
            return self._decode_native(mb)
        while True:
            st = self._mb_state(mb)
            if len(st.seqs) == 0:
                return None
            adv, src = self._advance(st, inflight)
            ctx_all = st.ctx + adv
            out_all = st.out_cnt + adv
            # a sequence the in-flight token completes (length budget / model length) is
            # not scheduled again
            keep = (adv == 0) | ((out_all < st.budget) & (ctx_all < self.max_model_len))
            idx = np.nonzero(keep)[0]
            if idx.size == 0:
                return None
            sid, ctx = st.sid[idx], ctx_all[idx]
            # blocks for the new tokens + their slots + the padded tables: one C++ call
            slots, tables, widest = self.bm.decode_prepare(sid, ctx, self.table_width)
            if widest is not None:
                break
            if not self._preempt(mb):
                return None
        n = len(sid)
        seeds = row_seeds(st.seed[idx], out_all[idx])
        feed = src[idx]
        meta = StepMeta(kind=DECODE, seq_ids=sid.tolist(), input_ids=st.last[idx],
                        positions=ctx - 1, slot_mapping=slots,
                        seq_lens=np.ones(n, np.int32), context_lens=ctx,
                        block_tables=tables, temperature=st.temp[idx], top_k=st.topk[idx],
                        top_p=st.topp[idx], seeds=seeds, microbatch=mb, step_id=self._step)
        meta.table_used = max(1, widest)
        meta.seq_ids_arr = sid
        if (feed >= 0).any():
            meta.feed_src = feed
        if self.state_slots is not None:
            meta.state_slots = self._slots_of([st.seqs[i] for i in idx.tolist()])
        return meta

    # ------------------------------------------------------------------ replay
    def replay_step(self, entries, want=None) -> StepMeta:
        """A step dictated from outside (trace replay, scoring): ``entries`` = [(request id,
        its next token ids)], all run as one batch — prompt portions of any length beside
        single tokens. A request is admitted at its first entry (blocks and, for stateful
        models, a state slot), may skip steps, and keeps what it holds until ``end_replay``.
        ``want`` = per entry, the indices among its new tokens whose logits are wanted; nothing
        is sampled. Same block manager, slot mapping, block tables and StepMeta as every
        other step."""
        self._step += 1
        picked, starts_l, lens_l = [], [], []
        for rid, toks in entries:
            toks = [int(t) for t in toks]
            if not toks:
                raise ValueError(f"replay entry '{rid}' brings no tokens")
            seq = self._replay.get(rid)
            if seq is None:
                seq = Sequence(seq_id=self._next_id, request_id=rid, prompt_ids=[],
                               params=SamplingParams(max_new_tokens=0, ignore_eos=True))
                self._next_id += 1
                seq.state = SeqState.PREFILLING
                self._replay[rid] = self.seqs[seq.seq_id] = seq
            if seq in picked:
                raise ValueError(f"replay request '{rid}' appears twice in one step")
            seq.prompt_ids.extend(toks)
            if not self.bm.ensure(seq.seq_id, seq.total_len):
                raise RuntimeError(f"cache pool exhausted at request '{rid}' "
                                   f"({seq.total_len} tokens, {self.bm.num_free} blocks free)")
            picked.append(seq)
            starts_l.append(seq.num_prefilled)
            lens_l.append(len(toks))
            seq.num_prefilled = seq.total_len
        S = len(picked)
        sid = np.fromiter((s.seq_id for s in picked), np.int64, S)
        starts = np.asarray(starts_l, np.int32)
        lens = np.asarray(lens_l, np.int32)
        T = int(lens.sum())
        ids = np.fromiter(itertools.chain.from_iterable(
            s.prompt_ids[st:st + n] for s, st, n in zip(picked, starts_l, lens_l)), np.int32, T)
        cu = np.zeros(S, np.int32)
        cu[1:] = np.cumsum(lens)[:-1]
        pos = (np.arange(T, dtype=np.int32) - np.repeat(cu - starts, lens)).astype(np.int32)
        width = -(-max(s.total_len for s in picked) // self.bs)
        temp, topk, topp, seeds = self._sampling_arrays(picked)
        meta = StepMeta(kind=PREFILL, seq_ids=sid.tolist(), input_ids=ids, positions=pos,
                        slot_mapping=self.bm.slot_mapping(sid, starts, lens), seq_lens=lens,
                        context_lens=starts + lens,
                        block_tables=self.bm.fill_tables(sid.tolist(), width), temperature=temp,
                        top_k=topk, top_p=topp, seeds=seeds, step_id=self._step,
                        seq_ids_arr=sid)
        meta.sample_mask = np.zeros(S, np.bool_)
        meta.state_slots = self._slots_of(picked)
        rows = [int(cu[i]) + int(k) for i, w in enumerate(want or []) for k in w]
        if any(not 0 <= k < lens_l[i] for i, w in enumerate(want or []) for k in w):
            raise ValueError("wanted index outside its entry's tokens")
        meta.logit_rows = np.asarray(rows, np.int64)
        return meta

    def end_replay(self, request_id: str) -> None:
        """Give back the blocks and the state slot of a replayed request."""
        seq = self._replay.pop(request_id, None)
        if seq is not None:
            self._finish(seq, "replay")
            self.seqs.pop(seq.seq_id, None)
            if seq in self.finished:
                self.finished.remove(seq)

    # ------------------------------------------------------------------ results
    def update(self, meta: StepMeta, tokens) -> List[Sequence]:
        """Apply sampled tokens of a finished step; returns sequences that finished."""
        tokens = np.asarray(tokens, dtype=np.int32).reshape(-1)
        mb = meta.microbatch
        core = getattr(meta, "core", None)
        if core is not None:
            st, steps, S = core
            if (st is self._state[mb] and st.core.steps == steps and st.core.rows == S
                    and tokens.shape[0] == S):
                return self._update_native(st, tokens, mb)
        st = self._state[mb] if meta.kind == DECODE else None
        if st is not None and len(st.seqs) == len(meta.seq_ids) and \
                np.array_equal(st.sid, meta.seq_ids_arr if meta.seq_ids_arr is not None
                               else np.asarray(meta.seq_ids, dtype=np.int64)):
            return self._update_fast(st, tokens, mb)
        self._drop_state(mb)
        return self._update_slow(meta, tokens)

    def _update_fast(self, st: _MBState, tokens: np.ndarray, mb: int) -> List[Sequence]:
        now = time.perf_counter()
        st.record(tokens)
        if st.first_pending:
            for i in np.nonzero(st.out_cnt == 0)[0].tolist():
                st.seqs[i].first_token_time = now
            st.first_pending = False
        st.last = tokens.copy()
        st.out_cnt += 1
        st.ctx += 1
        fin = st.out_cnt >= st.budget
        if self.eos is not None:
            fin_stop = st.eos_ok & (tokens == self.eos)
        else:
            fin_stop = np.zeros_like(fin)
        for i in st.stops:
            if int(tokens[i]) in st.seqs[i].params.stop_token_ids:
                fin_stop[i] = True
        fin_len = fin | (st.ctx >= self.max_model_len)
        done_mask = fin_len | fin_stop
        done_idx = np.nonzero(done_mask)[0]
        done = []
        if done_idx.size:
            idx = done_idx.tolist()
            st.flush_rows(idx)
            seqs = st.seqs
            for i in idx:
                s = seqs[i]
                self._mark_finished(s, "length" if fin_len[i] and not fin_stop[i] else "stop")
                done.append(s)
            if done_idx.size == len(seqs):
                self.running[mb] = []
                self._state[mb] = None
            else:
                st.compact(~done_mask)
                self.running[mb] = list(st.seqs)
        return done

    def _update_native(self, st: _MBCore, tokens: np.ndarray, mb: int) -> List[Sequence]:
        done_idx, stop = st.core.update(tokens)
        if st.first_rows:
            now = time.perf_counter()
            for i in st.first_rows:
                st.seqs[i].first_token_time = now
            st.first_rows = []
        done = []
        if done_idx.shape[0]:
            seqs = st.seqs
            idx = done_idx.tolist()
            if len(idx) > 8:          # many rows finish together: one history copy
                hist = st.core.history()[done_idx].tolist()
            else:
                hist = [st.core.row_history(i) for i in idx]
            for i, sf, h in zip(idx, stop.tolist(), hist):
                s = seqs[i]
                s.output_ids.extend(h)
                self._mark_finished(s, "stop" if sf else "length", free=False)
                done.append(s)
            self.bm.free_batch(np.fromiter((q.seq_id for q in done), np.int64, len(done)))
            if len(idx) == len(seqs):
                self.running[mb] = []
                self._state[mb] = None
            else:
                st.core.compact(done_idx)
                dropped = set(idx)
                st.seqs = [q for i, q in enumerate(seqs) if i not in dropped]
                self.running[mb] = list(st.seqs)
        return done

    def _update_slow(self, meta: StepMeta, tokens: np.ndarray) -> List[Sequence]:
        done = []
        now = time.perf_counter()
        touched = set()
        mask = meta.sample_mask
        for i, sid in enumerate(meta.seq_ids):
            seq = self.seqs.get(sid)
            if seq is None or seq.state != SeqState.RUNNING or (mask is not None and not mask[i]):
                continue
            if meta.step_id < seq.preempt_step:
                continue        # scheduled before the sequence was preempted: a stale token
            touched.add(seq.microbatch)
            t = int(tokens[i])
            seq.output_ids.append(t)
            if seq.first_token_time is None:
                seq.first_token_time = now
            p = seq.params
            reason = None
            if len(seq.output_ids) >= p.budget(seq.prompt_len):
                reason = "length"
            elif not p.ignore_eos and self.eos is not None and t == self.eos:
                reason = "stop"
            elif t in p.stop_token_ids:
                reason = "stop"
            elif seq.total_len >= self.max_model_len:
                reason = "length"
            if reason:
                self._finish(seq, reason)
                done.append(seq)
        for mb in touched:
            self._drop_state(mb)
        return done

    def pop_finished(self) -> List[Sequence]:
        out, self.finished = self.finished, []
        for s in out:
            self.seqs.pop(s.seq_id, None)
        return out
