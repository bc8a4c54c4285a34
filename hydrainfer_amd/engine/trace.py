"""Replaying a trace of token ids through a serving node, step by step, for the logits of chosen positions.

A trace step names, for every request that takes part, its next tokens and the positions among them whose logits are
wanted; nothing is sampled.  The replayer turns each piece into a TextFill instruction (Fill.logit_rows) at the end of
the request's instruction chain, parks the request on an AwaitTokens instruction between its pieces, and lets the node's
own step — scheduler, cache and state-slot managers, fill executor, model — run the batch.  `bin/trace_run` is the
command-line front of this class."""
import json
import sys
from typing import Dict, List, Optional

import torch

from hydrainfer_amd.engine.isa import AwaitTokens, InstructionListBuilder, TextFill
from hydrainfer_amd.engine.rcb import OutputTokenProcessor, RequestControlBlock, SamplingParameters
from hydrainfer_amd.engine.scheduler import BatchSchedulerConfig

BLOCK_SIZE = 16


class LogitsCollector(OutputTokenProcessor):
    def __init__(self):
        self.rows: List[torch.Tensor] = []

    def append_token_id(self, token_id, is_last_token=False):
        pass

    def append_logits(self, logits, instruction):
        self.rows.append(logits)

    def take(self) -> List[torch.Tensor]:
        rows, self.rows = self.rows, []
        return rows


class TraceReplayer:
    def __init__(self, language_model, dtype: torch.dtype, device, max_tokens: int, max_live_requests: int = 4):
        from hydrainfer_amd.engine.serve import build_node
        self.device = torch.device(device)
        shape = language_model.language_model.shape
        sched = BatchSchedulerConfig(priority="prefill", max_running_requests=max_live_requests, chunked_prefill=False,
                                     token_budgets=1 << 30, image_budgets=0)
        n_blocks = (int(max_tokens) + BLOCK_SIZE - 1) // BLOCK_SIZE
        self.node = build_node("EPD0", "EPD", language_model, None, shape, dtype, self.device, kv_blocks=n_blocks,
                               image_blocks=0, n_image_tokens=0, sched=sched, graph_decode=False)
        self.live: Dict[str, RequestControlBlock] = {}
        self.fed: Dict[str, int] = {}
        self.n_requests = 0

    @classmethod
    def from_checkpoint(cls, model_path: str, dtype: torch.dtype, device, max_tokens: int, **kw) -> "TraceReplayer":
        from hydrainfer_amd.model.registry import load_model
        lm, _ = load_model(model_path, dtype, device, vision=False)
        return cls(lm, dtype, device, max_tokens, **kw)

    def _piece(self, rid: str, tokens: List[int], want: List[int]):
        lo = self.fed.get(rid, 0)
        ids = list(range(lo, lo + len(tokens)))
        fill = TextFill(list(tokens), ids, list(ids), False, None, None)
        fill.logit_rows = list(want) or None
        self.fed[rid] = lo + len(tokens)
        return fill

    def step(self, entries: List[dict], end: List[str]) -> Optional[torch.Tensor]:
        """Runs one trace step; returns the wanted logits [n_wanted, vocab] (float32, on the device) in the order of the
        entries and of their `want` lists, or None if the step wants none."""
        parked = []
        for e in entries:
            rid, tokens = e["id"], e["tokens"]
            if not tokens:
                raise ValueError(f"request {rid}: an entry without tokens")
            fill, wait = self._piece(rid, tokens, e.get("want") or []), AwaitTokens()
            rcb = self.live.get(rid)
            if rcb is None:
                rcb = self.live[rid] = RequestControlBlock()
                rcb.request_id = self.n_requests
                self.n_requests += 1
                rcb.sampling_params = SamplingParameters(max_tokens=1 << 30)
                b = InstructionListBuilder()
                b.append(fill)
                b.append(wait)
                rcb.instructions = b.build_instruction_list()
                rcb.register_output_token_processor(LogitsCollector())
                self.node.add_request(rcb)
            else:
                rcb.instructions.extend(fill)
                rcb.instructions.extend(wait)
            parked.append((rcb, wait))
        self.node.step()
        for (rcb, wait), e in zip(parked, entries):
            if rcb.current_instruction() is not wait:
                raise RuntimeError(f"request {e['id']} did not run in its step (cache pool or state slots exhausted: "
                                   f"{len(self.node.kv_cache_block_manager.shared_cache.to_be_evicted)} blocks free)")
        rows = [r for rcb, _ in parked for r in rcb.output_token_processors[0].take()]
        done = [rid for rid in end if rid in self.live]
        for rid in done:
            rcb = self.live.pop(rid)
            self.fed.pop(rid, None)
            node = rcb.instructions.tail.prev
            assert isinstance(node, AwaitTokens)
            node.closed = True
        if done:
            self.node.step()       # the ended requests reach the end of their chains: blocks and state slots go back
        return torch.cat(rows, dim=0) if rows else None


def replay_stdin(replayer: TraceReplayer, out_dir: str, lines=None, report=None) -> None:
    """One JSON object a line: {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.  Writes <out_dir>/<n>.f32
    (little-endian float32 [wanted, vocab]) for a step that wants logits and prints `done <n>` after every step."""
    import os
    lines = sys.stdin if lines is None else lines
    report = report or (lambda text: (sys.stdout.write(text + "\n"), sys.stdout.flush()))
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = replayer.step(step.get("entries") or [], step.get("end") or [])
        if logits is not None:
            data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4")
            tmp = os.path.join(out_dir, f".{step['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
        report(f"done {step['step']}")
