"""The model as the engine runs it: embedding, a schedule of blocks, final
norm, head.  It is built from a ModelSpec alone; every stage is a part chosen
by the spec."""

from __future__ import annotations

import torch

from ..config.specs import ModelSpec
from ..parts.base import CompositeSpec, HiddenState, ParamSpec, Part, StateSpec, build_part


class DecoderModel:
    """Reference: shrike/models/qwen.py:153-192 (embedding, layers, final norm,
    selection of the wanted rows before the output matrix)."""

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        h = spec.hidden_size
        self.embedding = build_part("embedding", spec.embedding, h, spec.embed_name)
        self.blocks = [build_part("block", b, h, b.name) for b in spec.blocks]
        self.final_norm = build_part("norm", spec.final_norm, h, spec.final_norm_name)
        self.head = build_part("head", spec.head, h, spec.head_name)
        if spec.tie_word_embeddings:
            self.head.tie(self.embedding)
        # an embedding that depends on the token before keeps it per request, as mixers keep state
        spec_of = getattr(self.embedding, "cache_spec", None)
        self.embedding_state = spec_of() if spec_of is not None else None
        if self.embedding_state is not None and not isinstance(self.embedding_state, StateSpec):
            raise TypeError("an embedding's cache need must be a StateSpec")
        # some run adds the embedding's output to the stream again: it is kept
        self._keep_embedding = any(e.add_embedding for e in spec.schedule)
        self.stream_vectors: dict = {}
        # every run's result is kept and the stream that goes on is a weighted sum of them
        self._averaged = bool(spec.schedule) and spec.schedule[0].depth_average is not None
        self.depth_coefficients: list = []
        # the parts whose prepare() does something, in the order they run
        self._preparers = [p for p in self.parts() if type(p).prepare is not Part.prepare]

    def parts(self) -> list[Part]:
        """Every part of the model, blocks' own parts included, in running order."""
        out: list[Part] = [self.embedding]
        for block in self.blocks:
            out.append(block)
            out += list(getattr(block, "parts", ()))
        return out + [self.final_norm, self.head]

    # ------------------------------------------------------------------ weights

    def params(self) -> list[ParamSpec]:
        out = list(self.embedding.params())
        for block in self.blocks:
            out += block.params()
        out += [ParamSpec(name, (rows, self.spec.hidden_size), init="vector", keep_float32=True)
                for name, rows in self.spec.stream_vectors]
        if self._averaged:
            out += [ParamSpec(entry.depth_average, (pos + 2,), init="average", keep_float32=True)
                    for pos, entry in enumerate(self.spec.schedule)]
        return out + self.final_norm.params() + self.head.params()

    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph:
        every part says so, and a mixer with state of its own says that it
        reaches that state through the device-side slot indices."""
        for part in self.parts():
            if not part.graph_safe:
                return False
        for block in self.blocks:
            mixer = block.mixer
            need = mixer.cache_spec()
            needs = [s for _, s in need.parts] if isinstance(need, CompositeSpec) else [need]
            if any(isinstance(s, StateSpec) for s in needs) and not mixer.state_graph_safe:
                return False
        if self.embedding_state is not None and not getattr(self.embedding, "state_graph_safe", False):
            return False
        return True

    def launches_follow_shape(self) -> bool:
        """Whether every part says that its launches follow from a step's shape and
        launch key alone: the forward of such a model can be run again from a recorded
        list of launches for any later step of the same shape."""
        return all(part.launches_follow_shape for part in self.parts())

    def cache_specs(self) -> list:
        """Cache need of every schedule position (None for a position that
        reads another position's cache or whose mixer keeps nothing), and after
        them, where the embedding keeps state per request, one more entry for it
        (position len(schedule))."""
        out = []
        for entry in self.spec.schedule:
            mixer = self.blocks[entry.block].mixer
            out.append(None if entry.cache_of is not None else mixer.cache_spec())
        if self.embedding_state is not None:
            out.append(self.embedding_state)
        return out

    def load(self, tensors: dict[str, torch.Tensor], runtime) -> None:
        self.embedding.check(runtime)
        self.embedding.load(tensors, runtime)
        for block in self.blocks:
            block.check(runtime)
            block.load(tensors, runtime)
        self.stream_vectors = {name: tensors[name] for name, _rows in self.spec.stream_vectors}
        if self._averaged:
            self.depth_coefficients = [tensors[e.depth_average].contiguous() for e in self.spec.schedule]
            self._one = torch.ones(1, dtype=torch.float32, device=runtime.device)
        self.final_norm.load(tensors, runtime)
        self.head.check(runtime)
        self.head.load(tensors, runtime)

    # ------------------------------------------------------------------ forward

    def prepare(self, shape) -> None:
        """Lets every part that wants to decide its launches for the step and add
        its index arrays to the step's metadata."""
        for part in self._preparers:
            part.prepare(shape)

    def forward(self, ctx, caches) -> torch.Tensor:
        """Logits float32 [R, vocab] at ctx.out_rows.  `caches[i]` is the
        LayerCache of schedule position i."""
        if self.embedding_state is not None:
            hidden = HiddenState(self.embedding.forward(ctx, cache=caches[len(self.spec.schedule)]))
        else:
            hidden = HiddenState(self.embedding.forward(ctx))
        embedded = self.embedding.forward(ctx, into="embedded") if self._keep_embedding else None
        history = None
        if self._averaged:
            # slot 0: the embedding's output; slot k + 1: run k's working stream, which starts as
            # the average that run k - 1 left and ends as run k's result; the last slot: what
            # goes on to the final norm
            from ..kernels import ops

            runs = len(self.spec.schedule)
            history = ctx.buffer("stream_history", (runs + 2, ctx.num_tokens, self.spec.hidden_size), torch.float32)
            first = hidden.resid.view(1, ctx.num_tokens, self.spec.hidden_size)
            ops.mix_history(first, self._one, 1, history[0])
            ops.mix_history(first, self._one, 1, history[1])
        for pos, entry in enumerate(self.spec.schedule):
            if history is not None:
                hidden = HiddenState(history[pos + 1])
            if entry.add_embedding or entry.add_vector is not None:
                from ..kernels import ops

                hidden.settle(ctx)
                vector = None
                if entry.add_vector is not None:
                    vector = self.stream_vectors[entry.add_vector[0]][entry.add_vector[1]]
                ops.add_rows(hidden.resid, embedded if entry.add_embedding else None, vector)
                hidden.cast = None
            self.blocks[entry.block].forward(ctx, hidden, caches[pos])
            if history is not None:
                # the run's result is its stream plus what is pending; a pending output with a
                # layer norm of its own is normed and added by the averaging kernel itself
                norm = hidden.pending_norm
                if hidden.pending is not None and not (norm is not None and len(norm) == 3):
                    hidden.settle(ctx)
                ops.mix_history(history, self.depth_coefficients[pos], pos + 2, history[pos + 2],
                                delta=hidden.pending, dnorm=norm if hidden.pending is not None else None,
                                dtype=ctx.dtype)
                hidden.pending = hidden.pending_norm = None
        if history is not None:
            hidden = HiddenState(history[len(self.spec.schedule) + 1])
        rows = ctx.out_rows
        if rows.shape[0] == 0:
            return ctx.buffer("logits", (0, self.spec.vocab_size), torch.float32)
        x = self.final_norm.forward(ctx, hidden, rows=rows, write_resid=False)
        return self.head.forward(ctx, x)
