"""How a layer's parts are arranged around the residual stream."""

from __future__ import annotations

from .base import FeedForward, Mixer, Norm, Part


class PreNormBlock(Part):
    """h += mixer(norm_1(h)); h += ffn(norm_2(h)), h being the float32 residual stream.

    This is the reference's layer (mercury/model/qwen2.py:82-94) with its carried `residual`
    written as the running sum: the reference adds the previous output inside the next norm,
    here each part adds its output into h as it produces it.

    `names` gives the checkpoint sub-prefix of each part, e.g. ``{"mixer": "self_attn.",
    "ffn": "mlp.", "norm_mixer": "input_layernorm.", "norm_ffn": "post_attention_layernorm."}``.
    """

    def __init__(self, mixer: Mixer, ffn: FeedForward | None, norm_mixer: Norm,
                 norm_ffn: Norm | None, names: dict):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        self.names = dict(names)

    def _children(self):
        out = [("mixer", self.mixer), ("norm_mixer", self.norm_mixer)]
        if self.ffn is not None:
            out += [("ffn", self.ffn), ("norm_ffn", self.norm_ffn)]
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._children())

    def lowerable_with(self, state) -> bool:
        """Whether the host core can run the whole layer: every part hands over its work, and
        a mixer with state of its own says that its operations take the state tensor
        (`lowers_state`)."""
        if state is not None and not getattr(self.mixer, "lowers_state", False):
            return False
        return all(part.can_lower() for _, part in self._children())

    def lower(self, program, cache, state=None) -> None:
        self.norm_mixer.lower(program)
        if state is None:
            self.mixer.lower(program, cache)
        else:
            self.mixer.lower(program, cache, state)
        if self.ffn is not None:
            self.norm_ffn.lower(program)
            self.ffn.lower(program)

    def param_specs(self) -> dict:
        specs = {}
        for key, part in self._children():
            for name, spec in part.param_specs().items():
                specs[self.names[key] + name] = spec
        return specs

    def bind(self, params, dtype, device) -> None:
        for key, part in self._children():
            prefix = self.names[key]
            part.bind({n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)},
                      dtype, device)

    def prepare(self, max_positions: int, device) -> None:
        self.mixer.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        return sum(part.weight_bytes() for _, part in self._children())

    def forward(self, h, step, cache, state, dtype, pending=None):
        """Runs the layer on the stream h.  `pending` are partial sums [P, T, H] that still
        have to be added into h (the previous projection's, when it left them to its
        consumer); the return value is the same for whoever reads h next."""
        x = self.norm_mixer.forward(h, dtype, partials=pending)
        pending = self.mixer.forward(x, step, cache, state, h)
        if self.ffn is not None:
            x = self.norm_ffn.forward(h, dtype, partials=pending)
            pending = self.ffn.forward(x, step, h)
        return pending
