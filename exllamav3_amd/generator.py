"""
Token-level generation over a step-interface model (registry.load_model) and its SlotStateCache: jobs, a scheduler with continuous
batching, and sampling.

Scheduling.  One engine iteration is one model step.  Waiting jobs are admitted first: as many as fit the step's row budget and the
batch cap become ONE packed prompt step (unequal prompt lengths, no padding), and each receives a slot.  Otherwise every running job
advances by one token in one decode step, whatever step they were admitted in.  A job that ends (token budget, stop token) gives its
slot back at once and the next admission reuses it.

Decode steps as graphs.  On a GPU the decode step of a given batch size is captured into a hipGraph the second time that size occurs
(the first time runs eagerly, which is also the libraries' warm-up) and replayed from then on: the step's integers (tokens, slots,
positions) are copied into the captured step's own device buffer, everything else -- weights, cache buffers, scratch from the graph's
pool -- keeps its address.  A cache that grows moves its buffers, and the graphs are dropped.  Prompt steps run eagerly (their shapes
vary, and the experts of long prompts read their counts on the host).

Sampling.  Greedy when temperature is 0; otherwise temperature, top-k and top-p filtering on the float32 logits and one multinomial
draw per job from the job's own generator (so a job's tokens do not depend on what else is in the batch).
"""
from __future__ import annotations
from dataclasses import dataclass, field
import torch
from .state_cache import SlotStateCache


@dataclass
class SamplerSettings:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0


class Sampler:
    def __init__(self, settings: SamplerSettings, device):
        self.s = settings
        self.gen = None
        if settings.temperature > 0:
            self.gen = torch.Generator(device=device)
            self.gen.manual_seed(int(settings.seed))

    def sample(self, logits: torch.Tensor) -> int:
        """logits: float32 [vocab] on the device."""
        s = self.s
        if s.temperature <= 0:
            return int(torch.argmax(logits).item())
        l = logits / s.temperature
        if s.top_k and s.top_k < l.numel():
            kth = torch.topk(l, s.top_k).values[-1]
            l = torch.where(l < kth, torch.full_like(l, float("-inf")), l)
        p = torch.softmax(l, dim=-1)
        if s.top_p < 1.0:
            sp, si = torch.sort(p, descending=True)
            keep = (torch.cumsum(sp, 0) - sp) < s.top_p          # the smallest prefix whose mass reaches top_p
            sp = torch.where(keep, sp, torch.zeros_like(sp))
            p = torch.zeros_like(p).scatter_(0, si, sp)
        return int(torch.multinomial(p / p.sum(), 1, generator=self.gen).item())


@dataclass
class Job:
    prompt: list
    max_new_tokens: int = 16
    sampling: SamplerSettings = field(default_factory=SamplerSettings)
    stop_tokens: tuple = ()
    output: list = field(default_factory=list)
    slot: int | None = None
    done: bool = False
    _sampler: Sampler | None = None


class Generator:
    def __init__(self, model, cache: SlotStateCache | None = None, max_batch: int = 64, max_step_rows: int = 16384, graphs: bool | None = None):
        self.model = model
        self.cache = cache if cache is not None else model.new_cache()
        self.max_batch, self.max_step_rows = max_batch, max_step_rows
        self.waiting: list[Job] = []
        self.running: list[Job] = []
        self.graphs = (torch.device(model.device).type == "cuda") if graphs is None else graphs
        self._graphs: dict[int, tuple] = {}      # batch size -> (graph, its StepBatch, its logits)
        self._seen: set[int] = set()
        self._generation = self.cache.generation
        self.graph_replays = 0

    def _decode_step(self, entries) -> torch.Tensor:
        """One token per sequence: eager the first time a batch size occurs, captured the second time, replayed afterwards."""
        if not self.graphs:
            return self.model.step(self.cache.begin_step(entries), self.cache)
        self.cache.reserve(entries)                # a cache with pages may grow here: before the graphs' addresses are trusted
        if self._generation != self.cache.generation:
            self._graphs.clear(); self._seen.clear()
            self._generation = self.cache.generation
        b = len(entries)
        held = self._graphs.get(b)
        if held is not None:
            graph, sb, logits = held
            self.cache.begin_step(entries, into=sb)
            graph.replay()
            self.graph_replays += 1
            return logits
        sb = self.cache.begin_step(entries)
        if not sb.decode or b not in self._seen:
            self._seen.add(b)
            return self.model.step(sb, self.cache)
        # capture records the launches without running them; the replay right after is this step
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.step(sb, self.cache)
        self._graphs[b] = (graph, sb, logits)
        graph.replay()
        self.graph_replays += 1
        return logits

    def enqueue(self, job: Job) -> Job:
        if not job.prompt:
            raise RuntimeError("a job needs at least one prompt token")
        if any(t < 0 or t >= self.model.vocab for t in job.prompt):
            raise RuntimeError("prompt token out of the vocabulary")
        job._sampler = Sampler(job.sampling, self.model.device)
        self.waiting.append(job)
        return job

    def busy(self) -> bool:
        return bool(self.waiting or self.running)

    def _admit(self) -> list[Job]:
        batch, rows = [], 0
        while self.waiting and len(self.running) + len(batch) < self.max_batch:
            j = self.waiting[0]
            if batch and rows + len(j.prompt) > self.max_step_rows:
                break
            batch.append(self.waiting.pop(0)); rows += len(j.prompt)
        return batch

    def iterate(self) -> list[tuple[Job, int]]:
        """One model step; returns (job, new token) for every job that advanced."""
        new = self._admit()
        if new:
            for j in new:
                j.slot = self.cache.alloc()
            jobs, entries = new, [(j.slot, list(j.prompt)) for j in new]
        elif self.running:
            jobs, entries = list(self.running), [(j.slot, [j.output[-1]]) for j in self.running]
        else:
            return []
        if new:
            logits = self.model.step(self.cache.begin_step(entries), self.cache)
        else:
            logits = self._decode_step(entries)
        out = []
        for i, j in enumerate(jobs):
            t = j._sampler.sample(logits[i])
            j.output.append(t)
            out.append((j, t))
            if len(j.output) >= j.max_new_tokens or t in j.stop_tokens:
                j.done = True
        if new:
            self.running.extend(new)
        for j in [j for j in self.running if j.done]:
            self.cache.release(j.slot)
            j.slot = None
            self.running.remove(j)
        return out

    def generate(self, prompts: list[list[int]], max_new_tokens: int = 16, sampling: SamplerSettings | None = None, stop_tokens=()) -> list[list[int]]:
        jobs = [self.enqueue(Job(list(p), max_new_tokens, sampling or SamplerSettings(), tuple(stop_tokens))) for p in prompts]
        while self.busy():
            self.iterate()
        return [j.output for j in jobs]
