"""Serving of layer-list models (config.SeqModelConfig): recurrent and windowed layers, whose
per-sequence memory is a fixed-size state plus a bounded window of cache pages.

SeqEngine is the step function: a ragged batch (portions of prompts beside single decoded tokens)
goes through one native pass (model_runner.SeqModel -> sd_seq_model_forward) over the engine's
slot and page caches (kv_cache.SeqCache).  SeqWorker puts the worker surface the scheduler
drives (execute_model over ExecuteModelRequest, as SpecDecodeWorker has it) on top, with the
library's sampling kernels.  A recurrent state cannot be rolled back to an earlier token, so these
models are served without speculation: one token per sequence and step.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib, ops
from .kv_cache import PAGE, OutOfPages, SeqCache
from .model_runner import SeqModel
from .weights import SeqModelWeights


@dataclass
class SeqEngineConfig:
    max_seqs: int = 4            # sequence slots (live requests)
    max_tokens: int = 4096       # tokens the page pool holds (window layers), over all live requests
    max_seq_len: int = 0         # longest sequence; 0: max_tokens
    max_rows: int = 2048         # token rows per native pass; a larger step runs as several passes
    # Steps that bring one token for each of their requests (decoding) replay as one hipGraph per
    # (requests, wanted rows): the pass reads tokens, positions, slots and page tables from device
    # buffers at fixed addresses, so only their contents change between replays.  The first step
    # of a shape runs launch by launch, the second is captured.
    use_graph: bool = True
    graph_max_rows: int = 64

    @property
    def max_batch(self) -> int:  # the name the scheduler reads
        return self.max_seqs


@dataclass
class _Seq:
    slot: int
    n: int = 0                   # tokens computed so far
    last: int = -1               # the last token computed (-1: none yet): part of the sequence's state


class SeqEngine:
    def __init__(self, weights: SeqModelWeights, cfg: Optional[SeqEngineConfig] = None):
        if not ops.on_gpu():
            raise _lib.SdError("layer-list models run on the GPU library only")
        self.cfg = cfg or SeqEngineConfig()
        c = self.cfg
        if c.max_seqs < 1 or c.max_tokens < 1 or c.max_rows < 1:
            raise ValueError("max_seqs, max_tokens and max_rows must be positive")
        self.weights = weights
        self.model_cfg = weights.cfg
        self.device = weights.embed.device
        self.max_seq_len = c.max_seq_len = c.max_seq_len or c.max_tokens
        num_pages = (c.max_tokens + PAGE - 1) // PAGE
        self.cache = SeqCache(weights.cfg, weights.dtype, c.max_seqs, num_pages, self.max_seq_len, self.device)
        self.model = SeqModel(weights, self.cache)
        self.seqs: Dict[str, _Seq] = {}
        self.passes = 0
        self.stream = torch.cuda.Stream(device=self.device)   # (a capture needs a stream of its own)
        self._graphs: Dict[Tuple[int, int], dict] = {}
        self.graph_replays = 0

    # ------------------------------------------------------------------ requests
    def has(self, request_id: str) -> bool:
        return request_id in self.seqs

    def add(self, request_id: str) -> int:
        if request_id in self.seqs:
            raise KeyError(f"request {request_id} is live already")
        self.seqs[request_id] = _Seq(self.cache.slots.alloc())
        return self.seqs[request_id].slot

    def finish(self, request_id: str) -> None:
        """Gives the request's slot and pages back."""
        self.cache.release(self.seqs.pop(request_id).slot)

    def num_computed(self, request_id: str) -> int:
        return self.seqs[request_id].n

    @property
    def free_slots(self) -> int:
        return self.cache.slots.num_free

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[Tuple[str, Sequence[int], Sequence[int]]],
             layer_out: bool = False):
        """entries: (request id, its next tokens, indices among them whose logits are wanted).
        A request is admitted at its first entry.  Returns the wanted logits, f32 [n, vocab] on
        the device, in the order of the entries and of their indices (and, with layer_out, the
        residual after every layer run, [layer runs, rows, width]; a layer that runs several times
        over counts each time)."""
        plan = []
        seen = set()
        for rid, toks, want in entries:
            if rid in seen:
                raise ValueError(f"request {rid} appears twice in a step")
            seen.add(rid)
            if len(toks) < 1:
                raise ValueError(f"request {rid}: an entry needs at least one token")
            if any(w < 0 or w >= len(toks) for w in want):
                raise ValueError(f"request {rid}: wanted index outside its tokens")
            if rid not in self.seqs:
                self.add(rid)
            s = self.seqs[rid]
            if s.n + len(toks) > self.max_seq_len:
                raise OutOfPages(f"request {rid}: {s.n + len(toks)} tokens exceed max_seq_len {self.max_seq_len}")
            self.cache.ensure_capacity(s.slot, s.n + len(toks))
            plan.append((s, list(toks), list(want)))
        n_want = sum(len(w) for _, _, w in plan)
        V = self.model_cfg.vocab
        logits = torch.empty(n_want, V, dtype=torch.float32, device=self.device)
        total = sum(len(t) for _, t, _ in plan)
        if layer_out and total > self.cfg.max_rows:
            raise ValueError("layer_out needs a step of at most max_rows rows")
        trace = (torch.empty(self.model_cfg.n_runs, total, self.model_cfg.width, dtype=torch.float32,
                             device=self.device) if layer_out else None)
        # cut the step into passes of at most max_rows rows (an entry may span passes)
        done = [0] * len(plan)
        out_at = [0] * len(plan)
        acc = 0
        for i, (_, _, w) in enumerate(plan):
            out_at[i] = acc
            acc += len(w)
        torch.cuda.current_stream(self.device).synchronize()   # the caller's work on its own stream
        with torch.cuda.stream(self.stream):
            self._run_passes(plan, done, out_at, logits, trace)
        self.stream.synchronize()
        for s, t, _ in plan:
            s.n += len(t)
            s.last = int(t[-1])
        return (logits, trace) if layer_out else logits

    def _run_passes(self, plan, done, out_at, logits, trace) -> None:
        while any(done[i] < len(plan[i][1]) for i in range(len(plan))):
            room = self.cfg.max_rows
            toks: List[int] = []
            pos: List[int] = []
            slot: List[int] = []
            prev: List[int] = []
            ents: List[int] = []
            out_rows: List[int] = []
            out_dst: List[int] = []
            for i, (s, t, w) in enumerate(plan):
                if room == 0 or done[i] >= len(t):
                    continue
                lo = done[i]
                hi = min(len(t), lo + room)
                row0 = len(toks)
                ents += [s.slot, row0, hi - lo, s.n + lo]
                toks += t[lo:hi]
                pos += range(s.n + lo, s.n + hi)
                slot += [s.slot] * (hi - lo)
                prev += [t[lo - 1] if lo > 0 else s.last] + t[lo:hi - 1]
                for j, wi in enumerate(w):
                    if lo <= wi < hi:
                        out_rows.append(row0 + wi - lo)
                        out_dst.append(out_at[i] + j)
                room -= hi - lo
                done[i] = hi
            self._run_pass(toks, pos, slot, prev, ents, out_rows, out_dst, logits, trace)

    def _drop_graphs(self) -> None:
        lib = _lib.load()
        for g in self._graphs.values():
            if g["graph"] is not None:
                lib.sd_graph_destroy(g["graph"])
        self._graphs = {}

    def __del__(self):
        try:
            self._drop_graphs()
        except Exception:
            pass

    def _run_graph_pass(self, host, R, E, O, out_dst, logits) -> bool:
        """A decode-shaped pass through its graph; False if this shape's graph is not there yet."""
        V = self.model_cfg.vocab
        lib = _lib.load()
        g = self._graphs.get((R, O))
        if g is None:                       # first time: buffers; the pass itself runs launch by launch
            self._graphs[(R, O)] = {"batch": torch.empty(host.numel(), dtype=torch.int32, device=self.device),
                                    "logits": torch.empty(max(O, 1), V, dtype=torch.float32, device=self.device),
                                    "graph": None, "workspace": None}
            return False
        dev = g["batch"]
        if g["graph"] is None or g["workspace"] != self.model.workspace.data_ptr():
            if g["graph"] is not None:      # the workspace grew since: its address is in the graph
                lib.sd_graph_destroy(g["graph"])
                g["graph"] = None
            self.model._ensure_workspace(R, O)
            handle = C.c_void_p()
            stream = ops._stream()
            _lib.check(lib.sd_graph_begin(stream), "sd_graph_begin")
            try:
                self.model.forward(R, E, dev[0:R], dev[R:2 * R], dev[2 * R:3 * R], dev[4 * R:4 * R + 4 * E], O,
                                   dev[4 * R + 4 * E:] if O else None, g["logits"] if O else None, None,
                                   dev[3 * R:4 * R])
            finally:
                rc = lib.sd_graph_end(stream, C.byref(handle))
            _lib.check(rc, "sd_graph_end")
            g["graph"], g["workspace"] = handle, self.model.workspace.data_ptr()
        dev.copy_(host)
        _lib.check(lib.sd_graph_launch(g["graph"], ops._stream()), "sd_graph_launch")
        if O and out_dst == list(range(out_dst[0], out_dst[0] + O)):
            logits[out_dst[0]:out_dst[0] + O].copy_(g["logits"][:O])
        elif O:
            logits[torch.tensor(out_dst, device=self.device)] = g["logits"][:O]
        self.graph_replays += 1
        self.passes += 1
        return True

    def _run_pass(self, toks, pos, slot, prev, ents, out_rows, out_dst, logits, trace) -> None:
        R, E, O = len(toks), len(ents) // 4, len(out_rows)
        host = torch.tensor(toks + pos + slot + prev + ents + out_rows, dtype=torch.int32)
        if self.cfg.use_graph and trace is None and R == E and R <= self.cfg.graph_max_rows:
            if self._run_graph_pass(host, R, E, O, out_dst, logits):
                return
        dev = host.to(self.device)
        a = dev[0:R]
        b = dev[R:2 * R]
        c = dev[2 * R:3 * R]
        p = dev[3 * R:4 * R]
        e = dev[4 * R:4 * R + 4 * E]
        o = dev[4 * R + 4 * E:]
        contiguous_out = O > 0 and out_dst == list(range(out_dst[0], out_dst[0] + O))
        V = self.model_cfg.vocab
        if O == 0:
            dst = None
        elif contiguous_out:
            dst = logits[out_dst[0]:out_dst[0] + O]
        else:
            dst = torch.empty(O, V, dtype=torch.float32, device=self.device)
        self.model.forward(R, E, a, b, c, e, O, o if O else None, dst, trace, p)
        if O and not contiguous_out:
            logits[torch.tensor(out_dst, device=self.device)] = dst
        self.passes += 1


# --------------------------------------------------------------------------------- worker
@dataclass
class SeqWorkerConfig:
    model: SeqModelWeights
    max_num_seqs: int = 4
    max_model_len: int = 2048
    max_num_batched_tokens: int = 0   # page pool in tokens; 0: max_num_seqs * max_model_len
    seed: int = 0


class SeqWorker:
    """The worker surface of spec_decode_worker.SpecDecodeWorker for a layer-list model: one
    execute_model per scheduler step, prompts (whole, or in pieces through num_prompt_tokens)
    beside running sequences in one ragged batch, one sampled token per running sequence."""

    def __init__(self, config: SeqWorkerConfig):
        self.config = config
        self.engine: Optional[SeqEngine] = None
        self._req: Dict[str, dict] = {}
        self._admitted = 0

    def init_device(self) -> None:
        pass

    def load_model(self) -> None:
        c = self.config
        pool = c.max_num_batched_tokens or c.max_num_seqs * (-(-c.max_model_len // PAGE) * PAGE)
        self.engine = SeqEngine(c.model, SeqEngineConfig(max_seqs=c.max_num_seqs, max_tokens=pool,
                                                         max_seq_len=c.max_model_len))

    def _sample(self, logits: torch.Tensor, rids: List[str]) -> List[int]:
        V = logits.shape[1]
        if V % 4:
            # the sampling kernels read rows in 16-byte pieces: a vocabulary that is no multiple of
            # four is padded with columns that can never be chosen
            wide = torch.full((logits.shape[0], V + 4 - V % 4), float("-inf"), dtype=torch.float32, device=logits.device)
            wide[:, :V] = logits
            return [min(t, V - 1) for t in self._sample(wide, rids)]
        reqs = [self._req[r] for r in rids]
        temps = [r["sp"].temperature or 0.0 for r in reqs]
        if not any(t > 0 for t in temps):
            return ops.argmax_rows(logits).tolist()
        dev = logits.device
        probs = ops.softmax_rows(logits, torch.tensor(temps, dtype=torch.float32, device=dev))
        sps = [r["sp"] for r in reqs]
        if any(sp.top_k > 0 or sp.top_p < 1.0 or sp.min_p > 0.0 for sp in sps):
            ops.filter_probs(probs, torch.tensor([sp.top_k for sp in sps], dtype=torch.int32, device=dev),
                             torch.tensor([sp.top_p for sp in sps], dtype=torch.float32, device=dev),
                             torch.tensor([sp.min_p for sp in sps], dtype=torch.float32, device=dev))
        u = [ops.uniform24(r["seed"], r["draws"], 0) for r in reqs]
        for r in reqs:
            r["draws"] += 1
        return ops.sample_rows(probs, torch.tensor(u, dtype=torch.float32, device=dev)).tolist()

    def execute_model(self, req):
        from .spec_decode_worker import ModelRunnerOutput
        eng = self.engine
        for rid in req.finished_requests_ids:
            if rid in self._req:
                del self._req[rid]
                eng.finish(rid)
        entries, emit = [], []
        for g in req.seq_group_metadata_list:
            rid = g.request_id
            if g.is_prompt:
                if rid in self._req:
                    raise KeyError(f"request {rid} is running already")
                sp = g.sampling_params
                seed = sp.seed if sp.seed is not None else (self.config.seed * 1000003 + self._admitted)
                self._admitted += 1
                self._req[rid] = {"prompt": list(g.prompt_token_ids), "fed": 0, "last": None, "sp": sp,
                                  "seed": int(seed) & (2 ** 63 - 1), "draws": 0}
            st = self._req[rid]
            left = len(st["prompt"]) - st["fed"]
            if left > 0:                       # (the next piece of) the prompt
                n = min(left, g.num_prompt_tokens or left)
                toks = st["prompt"][st["fed"]:st["fed"] + n]
                st["fed"] += n
                last = st["fed"] == len(st["prompt"])
                entries.append((rid, toks, [n - 1] if last else []))
                emit.append(last)
            else:                              # a running sequence: its last token
                entries.append((rid, [st["last"]], [0]))
                emit.append(True)
        ids: List[str] = [e[0] for e in entries]
        sampled: List[List[int]] = [[] for _ in ids]
        if entries:
            logits = eng.step(entries)
            rows = [i for i, e in enumerate(emit) if e]
            if rows:
                toks = self._sample(logits, [ids[i] for i in rows])
                for i, t in zip(rows, toks):
                    sampled[i] = [int(t)]
                    self._req[ids[i]]["last"] = int(t)
        return ModelRunnerOutput(ids, {r: i for i, r in enumerate(ids)}, sampled)
