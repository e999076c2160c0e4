"""A model: parts built from a ModelSpec, weights bound to them, and the
forward pass over one step's batch.  Nothing here names an architecture."""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Tuple

import torch

from ..config.registry import load_config
from ..errors import ConfigError
from ..parts.base import Part, build_part
from ..parts.lazy import Normed
from ..weights.loader import WeightSpec, load_weights
from .batch import StepContext
from .runtime import Runtime
from .spec import ModelSpec, PartSpec


def _walk(part: Part):
    yield part
    for child in part.children():
        yield from _walk(child)


class _Bound:
    """A built part with the file names of its tensors."""
    def __init__(self, part: Part, spec: PartSpec):
        self.part, self.spec = part, spec

    def names(self) -> Dict[str, Tuple[str, WeightSpec]]:
        return {local: (self.spec.prefix + self.spec.rename.get(local, local), ws)
                for local, ws in self.part.weight_specs().items()}


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = _Bound(build_part("embedding", spec.embedding), spec.embedding)
        self.final_norm = _Bound(build_part("norm", spec.final_norm), spec.final_norm)
        self.head = _Bound(build_part("head", spec.head), spec.head)
        self.layers: List[Part] = []
        self._layer_bound: List[List[_Bound]] = []
        for ls in spec.layers:
            mixer = _Bound(build_part("mixer", ls.mixer), ls.mixer)
            ffn = _Bound(build_part("feedforward", ls.ffn), ls.ffn)
            n1 = _Bound(build_part("norm", ls.mixer_norm), ls.mixer_norm)
            n2 = _Bound(build_part("norm", ls.ffn_norm), ls.ffn_norm)
            block = build_part("block", PartSpec(ls.block, dict(
                mixer=mixer.part, ffn=ffn.part, mixer_norm=n1.part, ffn_norm=n2.part)))
            self.layers.append(block)
            self._layer_bound.append([n1, mixer, n2, ffn])
        self.schedule = list(spec.schedule)
        for e in self.schedule:
            if not (0 <= e.layer < len(self.layers)):
                raise ConfigError(f"schedule names layer {e.layer}, the model has {len(self.layers)}")
        self.vocab_size = spec.vocab_size
        self.hidden_size = spec.hidden_size
        self.max_seq_len = spec.max_seq_len
        self.rt: Optional[Runtime] = None

    def all_parts(self) -> List[Part]:
        """Every part of the model, nested ones included: embedding, each layer's block with its norms,
        mixer and feed-forward, final norm, head."""
        tops = [self.embedding.part, *self.layers, self.final_norm.part, self.head.part]
        return [p for top in tops for p in _walk(top)]

    # ---- weights ------------------------------------------------------------
    def _all_bound(self) -> List[_Bound]:
        out = [self.embedding]
        for group in self._layer_bound:
            out.extend(group)
        out.extend([self.final_norm, self.head])
        return out

    def expected_weights(self) -> Dict[str, WeightSpec]:
        """File tensor name -> what the configuration needs of it."""
        out: Dict[str, WeightSpec] = {}
        for b in self._all_bound():
            for local, (name, ws) in b.names().items():
                if name in out and out[name].shape != ws.shape:
                    raise ConfigError(f"tensor '{name}' is wanted in two shapes")
                out[name] = ws
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        """Place the loaded tensors on the device and hand each part its own."""
        self.rt = rt
        placed: Dict[str, torch.Tensor] = {}
        cuda = rt.device.type == "cuda"
        before = torch.cuda.memory_allocated(rt.device) if cuda else 0

        def get(name: str) -> Optional[torch.Tensor]:
            if name not in placed and name in tensors:
                placed[name] = rt.place_weight(tensors[name])
            return placed.get(name)

        for b in self._all_bound():
            mine = {}
            for local, (name, ws) in b.names().items():
                t = get(name)
                if t is None:
                    tied = getattr(b.part, "tied_to", None)
                    t = get(tied) if tied else None
                    if t is None:
                        raise ConfigError(f"tensor '{name}' was not loaded")
                mine[local] = t
            b.part.bind(mine, rt)
        # the tensors as loaded, and what they take on the device once the parts have packed them and what
        # nobody holds any more has gone (a linear map's weight is kept once, in the order its kernels read)
        self.weight_bytes = sum(t.numel() * t.element_size() for t in placed.values())
        placed.clear()
        tensors = mine = None
        self.device_weight_bytes = torch.cuda.memory_allocated(rt.device) - before if cuda else self.weight_bytes

    # ---- cache --------------------------------------------------------------
    def cache_streams(self) -> Dict[Hashable, object]:
        """Cache stream id -> spec, from the schedule: the entry that writes a
        stream decides its spec; an entry may only read a stream that some
        entry writes."""
        streams: Dict[Hashable, object] = {}
        for e in self.schedule:
            if e.cache is None or not e.writes:
                continue
            spec = self.layers[e.layer].mixer.cache_spec()
            if e.cache in streams and streams[e.cache] != spec:
                raise ConfigError(f"cache stream {e.cache!r} is written with two different specs")
            streams[e.cache] = spec
        layouts: Dict[Hashable, object] = {}
        for e in self.schedule:
            if e.cache is None:
                continue
            if e.cache not in streams:
                raise ConfigError(f"schedule entry for layer {e.layer} reads cache stream {e.cache!r}, "
                                  "which no entry writes")
            mixer = self.layers[e.layer].mixer
            if mixer.cache_spec() != streams[e.cache]:
                raise ConfigError(f"layer {e.layer} uses cache stream {e.cache!r} with another spec than its writer")
            layout = mixer.cache_layout() if hasattr(mixer, "cache_layout") else None
            if layouts.setdefault(e.cache, layout) != layout:
                raise ConfigError(f"layers sharing cache stream {e.cache!r} keep a head's dimensions in "
                                  "different orders (their position encodings or dtypes differ)")
        return streams

    # ---- what a step costs -----------------------------------------------------
    def step_work(self, batch, n_logits: int, elem: int):
        """(floating-point operations, bytes that have to be read at least) of one step over ``batch``
        (a HostBatch) with logits at ``n_logits`` rows: every weight the step uses once, the cache of
        the live requests, as the parts state them; a layer that the schedule names twice counts twice."""
        flops, nbytes = self.embedding.part.step_work(batch, batch.n_tokens, elem)
        for e in self.schedule:
            f, b = self.layers[e.layer].step_work(batch, batch.n_tokens, elem)
            flops, nbytes = flops + f, nbytes + b
        for part in (self.final_norm.part, self.head.part):
            f, b = part.step_work(batch, n_logits, elem)
            flops, nbytes = flops + f, nbytes + b
        return flops, nbytes

    def working_bytes(self, rows: int, n_logits: int, elem: int) -> int:
        """Device bytes a step of ``rows`` rows with logits at ``n_logits`` of them needs beyond weights and cache, as
        the parts state it: the float residual stream and a normed copy of it, the layer that needs most (one
        layer's activations are given back before the next runs), and the float logits."""
        layer = max((part.working_bytes_per_row(elem) for part in self.layers), default=0.0)
        head = self.final_norm.part.working_bytes_per_row(elem) + self.hidden_size * elem
        per_row = self.hidden_size * (4 + 4 + elem) + self.embedding.part.working_bytes_per_row(elem) + layer
        return int(rows * per_row + n_logits * (head + 4 * self.vocab_size))

    # ---- forward ------------------------------------------------------------
    def forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """Run the batch through every schedule entry; float32 logits at the
        wanted rows ([n_logits, vocab]), or None if none are wanted."""
        x = self.embedding.part.forward(ctx)
        ctx.handoff.end_step()
        for i, e in enumerate(self.schedule):
            layer = self.layers[e.layer]
            following = self.layers[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
            ctx.handoff.begin_entry(layer, following, ctx.n_tokens)
            layer.forward(x, ctx, ctx.cache(e.cache), e.writes)
        ctx.handoff.end_step()
        if ctx.n_logits == 0:
            return None
        norm, head = self.final_norm.part, self.head.part
        if getattr(head, "accepts_lazy_norm", False):
            return head.forward(Normed(x, norm, ctx, rows=ctx.logit_rows, n_rows=ctx.n_logits))
        return head.forward(norm.forward(x, ctx, rows=ctx.logit_rows, n_rows=ctx.n_logits))


def expected_weights(spec: ModelSpec) -> Dict[str, WeightSpec]:
    return Model(spec).expected_weights()


def load_model(model_dir: str, dtype, device="cuda:0") -> Tuple[Model, object]:
    """(model with weights on the device, typed configuration) of a model folder."""
    from .runtime import parse_dtype
    arch, cfg = load_config(model_dir)
    model = Model(arch.describe(cfg))
    tensors = load_weights(model_dir, model.expected_weights(), ignore=arch.ignored_tensors)
    model.bind(tensors, Runtime(torch.device(device), parse_dtype(dtype)))
    return model, cfg
