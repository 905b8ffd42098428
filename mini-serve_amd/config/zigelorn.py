"""Typed configuration of the Zigelorn decoder, read from its own ``config.json`` keys. The reference has no such
architecture.

``config.json``: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list in which every
entry names its mixer (``type``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, or null for
none). Layer ``i``'s tensors start with ``l<i>.``. An entry with ``weights_of: j`` has no tensors: it runs layer ``j``'s
weights (mixer, feed-forward and norms) over a cache and state of its own, and the rest of its entry equals layer ``j``'s
(``j`` may come before or after it; where ``j`` runs another layer's weights in turn, that layer's are meant).

A layer is ``x += N1b(mixer(N1(x)))``, then ``x += N2b(ff(N2(x)))``, every ``N`` an RMS norm whose stored weight lies
around zero (``y / rms(y) * (1 + w)``; tensors ``norm1 norm1b norm2 norm2b``). The mixers:

* ``attention`` (``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional ``rot`` and ``mask``; tensors ``mix.q q.b k
  k.b q.norm k.norm g o``): grouped-query attention whose values are the keys as projected (bias included, before norm
  and rotation; ``vdim`` equals ``dim``). One RMS norm with a plain weight over a token's whole query projection and one
  over its key projection; then ``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``, ``original``, ``fast``,
  ``slow``) turns the first ``dims`` elements of each query and key head, halves paired, by
  ``position * base ** (-2i / dims)``; with ``scaling`` the frequencies between the indices at which a wave makes ``fast``
  and ``slow`` turns within ``original`` positions are blended towards ``f / factor`` and cosines and sines are multiplied
  by ``0.1 ln(factor) + 1``. A query sees the last ``mask.size`` tokens, itself included (no ``mask``: every earlier
  token). Head ``h``'s output is multiplied by ``sigmoid(g x)_h``.
* ``retention`` (``heads``, ``dim``, ``vdim``, ``decay`` (one per head), optional ``rot``; tensors ``mix.q k v g o``):
  ``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head, q and k turned as above, k times ``dim ** -0.5``
  behind the rotation; every head's output divided by its root mean square, times ``silu(g x)``.
* ``wkv`` (``heads``, ``dim``; tensors ``mix.mu.r k v g w``, ``mix.r k v g w1 w2 w0 u norm o``): each of r, k, v, the gate
  and the decay reads ``x + (x' - x) mu_s`` with ``x'`` the previous token's input (zeros for the first token);
  ``w = exp(-exp(w2 tanh(w1 mix_w) + w0))`` per key channel; ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then
  ``S_t = diag(w_t) S_(t-1) + k_t v_t^T``; every head's output divided by its root mean square, times ``norm``, times
  ``silu(g mix_g)``. How wide ``w1`` is no key says: the tensors do (``mixer.rank``, optional, states it for the
  random-weights mode).

Feed-forwards: ``kind: dense`` (``ff``; tensors ``mlp.up down``), ``down(gelu_tanh(up x))``; ``kind: moe`` (``router.experts``,
``router.top``, optional ``router.identity`` and ``router.groups`` with ``count`` and ``keep``, ``expert.ff``; tensors
``mlp.router``, ``mlp.correction``, ``mlp.e<j>.up down``): the router has ``experts + identity`` outputs, the last
``identity`` of which stand for experts that return their input; scores are the softmax over all outputs; the choice goes
by score plus ``correction``, within the ``keep`` best of ``count`` groups of neighbouring outputs (a group's score: its
largest choice score); the ``top`` chosen experts (``down(relu(up x)^2)``) are weighed by their scores as they stand. The
final norm is ``final.norm``; the head is the embedding table ``embed``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass

from .registry import register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunEntry

MIXER_TYPES = ("attention", "retention", "wkv")
MLP_KINDS = ("dense", "moe")


def _need(d, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ValueError(f"{where} must be an object, got {d!r}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise KeyError(f"config.json lacks {missing} in {where}")


def _positive_int(d: dict, key: str, where: str) -> int:
    v = d[key]
    if not isinstance(v, int) or isinstance(v, bool) or v < 1:
        raise ValueError(f"{where}.{key} must be a positive integer, got {v!r}")
    return v


def _check_rot(rot, dim: int, where: str) -> None:
    _need(rot, ("base", "dims"), where)
    dims = rot["dims"]
    if not isinstance(dims, int) or isinstance(dims, bool) or dims % 2 or not 2 <= dims <= dim:
        raise ValueError(f"{where}.dims must be even and at most dim, got {dims!r}")
    if not float(rot["base"]) > 1:
        raise ValueError(f"{where}.base must be larger than one")
    sc = rot.get("scaling")
    if sc:
        _need(sc, ("factor", "original", "fast", "slow"), f"{where}.scaling")
        if not all(float(sc[k]) > 0 for k in ("factor", "original", "fast", "slow")):
            raise ValueError(f"{where}.scaling: factor, original, fast and slow must be positive")


@register_architecture("Zigelorn")
@dataclass(frozen=True)
class ZigelornConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple  # of dicts as in config.json: {"type", "mixer", "mlp"[, "weights_of"]}

    @classmethod
    def from_dict(cls, cfg: dict) -> "ZigelornConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "norm")
        if not isinstance(cfg["layers"], (list, tuple)) or not cfg["layers"]:
            raise ValueError("layers must be a non-empty list")
        out = cls(
            vocab=_positive_int(cfg, "vocab", "config.json"),
            width=_positive_int(cfg, "width", "config.json"),
            eps=float(cfg["norm"]["eps"]),
            layers=tuple(copy.deepcopy(layer) for layer in cfg["layers"]),
        )
        out.validate()
        return out

    def validate(self) -> None:
        if not self.eps >= 0:
            raise ValueError(f"norm.eps must not be negative, got {self.eps}")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise NotImplementedError(f"{where}.type {kind!r} is not supported, expected one of {MIXER_TYPES}")
            mw = f"{where}.mixer"
            _need(m, ("heads", "dim"), mw)
            for k in ("heads", "dim"):
                _positive_int(m, k, mw)
            if kind == "attention":
                _need(m, ("kv_heads", "scale"), mw)
                _positive_int(m, "kv_heads", mw)
                if m["heads"] % m["kv_heads"]:
                    raise ValueError(f"{mw}: {m['heads']} heads are no multiple of {m['kv_heads']} kv_heads")
                if m.get("vdim", m["dim"]) != m["dim"]:
                    raise ValueError(f"{mw}: the values are the keys, so vdim {m['vdim']!r} must equal dim {m['dim']}")
                if not float(m["scale"]) > 0:
                    raise ValueError(f"{mw}.scale must be positive")
                if m.get("mask"):
                    _need(m["mask"], ("size",), f"{mw}.mask")
                    _positive_int(m["mask"], "size", f"{mw}.mask")
            elif kind == "retention":
                _need(m, ("vdim", "decay"), mw)
                _positive_int(m, "vdim", mw)
                decay = m["decay"]
                if not isinstance(decay, (list, tuple)) or len(decay) != m["heads"] or not all(0.0 <= float(d) <= 1.0 for d in decay):
                    raise ValueError(f"{mw}.decay must hold one number in [0, 1] per head, got {decay!r}")
            elif m.get("rank") is not None:
                _positive_int(m, "rank", mw)
            if kind != "wkv" and m.get("rot"):
                _check_rot(m["rot"], m["dim"], f"{mw}.rot")
            if layer.get("weights_of") is not None:
                root = self.source(i)
                if self.layers[root]["type"] != kind:
                    raise ValueError(f"{where} is a {kind!r} layer but runs the weights of layer {root}, a {self.layers[root]['type']!r} layer")
            mlp = layer.get("mlp")
            if mlp:
                fw = f"{where}.mlp"
                _need(mlp, ("kind",), fw)
                if mlp["kind"] not in MLP_KINDS:
                    raise NotImplementedError(f"{fw}.kind {mlp['kind']!r} is not supported, expected one of {MLP_KINDS}")
                if mlp["kind"] == "dense":
                    _need(mlp, ("ff",), fw)
                    _positive_int(mlp, "ff", fw)
                else:
                    _need(mlp, ("router", "expert"), fw)
                    r = mlp["router"]
                    _need(r, ("experts", "top"), f"{fw}.router")
                    _need(mlp["expert"], ("ff",), f"{fw}.expert")
                    _positive_int(mlp["expert"], "ff", f"{fw}.expert")
                    n = _positive_int(r, "experts", f"{fw}.router")
                    top = _positive_int(r, "top", f"{fw}.router")
                    identity = r.get("identity") or 0
                    if not isinstance(identity, int) or isinstance(identity, bool) or identity < 0:
                        raise ValueError(f"{fw}.router.identity must be a non-negative integer, got {identity!r}")
                    outputs, choosable = n + identity, n + identity
                    g = r.get("groups")
                    if g:
                        _need(g, ("count", "keep"), f"{fw}.router.groups")
                        count = _positive_int(g, "count", f"{fw}.router.groups")
                        keep = _positive_int(g, "keep", f"{fw}.router.groups")
                        if outputs % count or keep > count:
                            raise ValueError(f"{fw}.router.groups: {outputs} router outputs in {count} groups of which {keep} are kept")
                        choosable = outputs // count * keep
                    if top > choosable:
                        raise ValueError(f"{fw}.router: top {top} of {choosable} outputs that can be chosen")

    def source(self, i: int) -> int:
        """The layer whose tensors layer ``i`` runs: itself, or what its ``weights_of`` leads to."""
        seen = {i}
        while self.layers[i].get("weights_of") is not None:
            j = self.layers[i]["weights_of"]
            if not isinstance(j, int) or isinstance(j, bool) or not 0 <= j < len(self.layers):
                raise ValueError(f"layers[{i}].weights_of must be the number of a layer, got {j!r}")
            if j in seen:
                raise ValueError(f"layers[{i}].weights_of leads back to layer {j}: no layer of the chain has tensors")
            seen.add(j)
            i = j
        return i

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back as this configuration."""
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [copy.deepcopy(layer) for layer in self.layers]}

    # ------------------------------------------------------------------ lowering

    def _norm(self, tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": self.width, "eps": self.eps, "tensor": tensor, "offset": 1.0})

    @staticmethod
    def _position(rot) -> PartSpec | None:
        if not rot:
            return None
        sc = rot.get("scaling")
        scaling = None if not sc else {"kind": "turn_ramp", "factor": float(sc["factor"]), "original": float(sc["original"]),
                                       "fast": float(sc["fast"]), "slow": float(sc["slow"])}
        return PartSpec("rotary", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "pairing": "halves", "scaling": scaling})

    def _mixer(self, kind: str, m: dict) -> PartSpec:
        if kind == "attention":
            mask = m.get("mask")
            return PartSpec("gqa_attention", {
                "prefix": "mix.", "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                "head_dim": m["dim"], "value_dim": m["dim"], "scale": float(m["scale"]), "window": int(mask["size"]) if mask else 0,
                "qk_norm": "projection", "qk_norm_eps": self.eps, "exact_weights": True, "bias": True, "values_are_keys": True,
                "head_gate": True, "position": self._position(m.get("rot")),
                "names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_bias": "q.b", "k_bias": "k.b",
                          "gate": "g"}})
        if kind == "retention":
            return PartSpec("decay_linear_attention", {
                "prefix": "mix.", "hidden_size": self.width, "num_heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
                "eps": self.eps, "decay": tuple(float(d) for d in m["decay"]), "activation": None, "k_scale": float(m["dim"]) ** -0.5,
                "norm_group": "head", "norm_weight": False, "gate_activation": "silu", "position": self._position(m.get("rot"))})
        return PartSpec("wkv", {"prefix": "mix.", "hidden_size": self.width, "num_heads": m["heads"], "head_dim": m["dim"],
                                "eps": self.eps, "decay_rank": m.get("rank")})

    def _feed_forward(self, mlp: dict | None) -> PartSpec:
        if not mlp:
            return PartSpec("none")
        if mlp["kind"] == "dense":
            return PartSpec("dense_mlp", {"prefix": "mlp.", "hidden_size": self.width, "intermediate_size": int(mlp["ff"]),
                                          "activation": "gelu_tanh", "names": {"up": "up", "down": "down"}})
        r = mlp["router"]
        g = r.get("groups") or {}
        return PartSpec("moe_mlp", {
            "prefix": "mlp.", "hidden_size": self.width, "intermediate_size": int(mlp["expert"]["ff"]),
            "num_experts": int(r["experts"]), "top": int(r["top"]), "activation": "relu_squared", "gated": False,
            "scoring": "softmax", "router_bias": True, "identity": int(r.get("identity") or 0),
            "groups": int(g.get("count") or 1), "keep_groups": int(g.get("keep") or g.get("count") or 1),
            "names": {"router": "router", "router_bias": "correction", "expert": "e{}.", "up": "up", "down": "down"}})

    def to_spec(self) -> ModelSpec:
        w = self.width
        layers, index = [], {}
        for i, layer in enumerate(self.layers):
            if layer.get("weights_of") is not None:
                continue
            mlp = layer.get("mlp")
            block = PartSpec("sandwich", {
                "mixer_norm": self._norm("norm1"), "mixer_out_norm": self._norm("norm1b"),
                "ffn_norm": self._norm("norm2") if mlp else None, "ffn_out_norm": self._norm("norm2b") if mlp else None,
                "spare": None if mlp else {"norm2": w, "norm2b": w}})
            index[i] = len(layers)
            layers.append(LayerSpec(f"l{i}.", block, self._mixer(layer["type"], layer["mixer"]), self._feed_forward(mlp)))
        # every entry runs over a cache and state of its own, whosever weights it runs
        order = [RunEntry(index[self.source(i)], i) for i in range(len(self.layers))]
        return ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=w,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "width": w, "tensor": "embed"}),
            layers=tuple(layers),
            run_order=tuple(order),
            final_norm=self._norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "width": w, "tensor": "head", "tied_to": "embed"}),
            max_position=None,
        )
