"""Weights by tensor name: checking a file against what the model asks for, then loading.

A model says what it needs as ``{name: ParamSpec}``.  A *source* hands tensors out by name;
:class:`SafetensorsSource` reads a model folder, :class:`RandomSource` draws them from a seed.
Before anything is loaded the whole request is checked, and every fault (missing tensors,
tensors nobody asked for, wrong shapes, wrong kinds) comes back in ONE :class:`WeightError`;
the reference stops at the first missing name
(reference: src/SharpInference.Engine/ForwardPass.cs:2301-2306).

Storage policy: 16-bit floats are kept as bfloat16; a tensor stored in 32-bit floats stays
float32; integer tables become int32.  In float32 mode every float tensor is widened to
float32 (exact for bfloat16 values).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple

import torch

from . import safetensors_io as st

INIT_NORMAL, INIT_NORM_WEIGHT, INIT_INT = "normal", "norm_weight", "int"


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    init: str = INIT_NORMAL      # how random mode fills it: N(0, std) | U(0.9, 1.1) | integers
    kind: str = "float"          # "float" or "int"


class WeightError(ValueError):
    """All faults of a weight file at once."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[str], wrong_kind: List[str],
                 where: str = ""):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_kind = list(wrong_shape), list(wrong_kind)
        lines = [f"weights{' in ' + where if where else ''} do not fit the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shape ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if wrong_kind:
            lines.append(f"  wrong kind ({len(wrong_kind)}): " + "; ".join(wrong_kind))
        super().__init__("\n".join(lines))


def check_specs(specs: Dict[str, ParamSpec], available: Dict[str, Tuple[Tuple[int, ...], torch.dtype]],
                where: str = "") -> None:
    missing = sorted(n for n in specs if n not in available)
    unexpected = sorted(n for n in available if n not in specs)
    wrong_shape, wrong_kind = [], []
    for n, spec in sorted(specs.items()):
        if n not in available:
            continue
        shape, dtype = available[n]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append(f"{n}: expected {list(spec.shape)}, found {list(shape)}")
        is_float = dtype.is_floating_point
        if (spec.kind == "float") != is_float:
            wrong_kind.append(f"{n}: expected {spec.kind}, found {dtype}")
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightError(missing, unexpected, wrong_shape, wrong_kind, where)


def storage_dtype(stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    """What a tensor stored as `stored` becomes in a model computing in `compute`."""
    if not stored.is_floating_point:
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


# ---------------------------------------------------------------------------
class TensorSource:
    """Hands tensors out by name, already on `device` and in their storage dtype."""

    def available(self) -> Dict[str, Tuple[Tuple[int, ...], torch.dtype]]:
        raise NotImplementedError

    def get(self, name: str) -> torch.Tensor:
        raise NotImplementedError

    where = ""


class SafetensorsSource(TensorSource):
    def __init__(self, model_dir: str, compute_dtype: torch.dtype, device):
        self.where = model_dir
        self.entries = st.index_folder(model_dir)
        self.compute_dtype = compute_dtype
        self.device = torch.device(device)

    def available(self):
        return {n: (e.shape, e.dtype) for n, e in self.entries.items()}

    def get(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        host = st.read_tensor(e)
        want = storage_dtype(e.dtype, self.compute_dtype)
        if host.dtype != want:
            host = host.to(want)
        return host.to(self.device)


class LayoutAdapter(TensorSource):
    """Presents a checkpoint that is laid out otherwise under the names and shapes the model asks
    for.  Nothing here knows a model: the adaptations are found from the names and shapes alone.

    * A container prefix: a multimodal file keeps the text decoder under a prefix (for instance
      ``language_model.``).  If a wanted name is absent but ``prefix + name`` exists for one common
      prefix, names are read through it, and tensors outside the prefix (another tower's) are not
      the decoder's business: they are neither loaded nor reported as unexpected.
    * Fused expert matrices: ``X.gate_up_proj`` in place of ``X.gate_proj`` and ``X.up_proj``.  The
      name decides the order of the axes: a stacked tensor without a ``.weight`` suffix holds
      ``[E, in, 2 * out]`` (gate columns first), and the ``down_proj`` stored beside it holds
      ``[E, in, out]``; a fused ``….weight`` holds ``[2 * out, in]`` as a linear layer does.  Where
      the name does not decide, the shape may (a transposed stack whose two sizes differ); where
      neither does, the tensor is left as it is and reported with its shape.
    The reference does the like when it slices an expert out of a packed tensor and ties a missing
    head to the embedding (reference: src/SharpInference.Engine/ForwardPass.cs:2105-2113, 410-413).
    No published checkpoint could be read where this was written: the adaptations are tested on
    files written in those layouts by the tests."""

    def __init__(self, inner: TensorSource, specs: Dict[str, ParamSpec]):
        self.inner = inner
        self.where = inner.where
        have = inner.available()
        self.prefix = self._find_prefix(specs, have)
        self._plan: Dict[str, tuple] = {}
        self._avail: Dict[str, Tuple[Tuple[int, ...], torch.dtype]] = {}
        used = set()
        for name, spec in specs.items():
            src = self.prefix + name
            want = tuple(spec.shape)
            if src in have:
                shape, dtype = tuple(have[src][0]), have[src][1]
                swapped = len(want) == 3 and shape == (want[0], want[2], want[1])
                beside_fused = self._fused_sibling(name) is not None and self.prefix + self._fused_sibling(name) in have
                if swapped and (beside_fused or want[1] != want[2]):
                    self._plan[name] = ("transpose", src)
                    self._avail[name] = (want, dtype)
                else:
                    self._plan[name] = ("plain", src)
                    self._avail[name] = (shape, dtype)
                used.add(src)
                continue
            fused = self._fused_source(name)
            if fused and self.prefix + fused[0] in have:
                fsrc, half = self.prefix + fused[0], fused[1]
                shape, dtype = have[fsrc]
                how = self._split_plan(tuple(shape), want, stacked_in_out=not fsrc.endswith(".weight"))
                if how is not None:
                    self._plan[name] = ("split", fsrc, half, how)
                    self._avail[name] = (want, dtype)
                    used.add(fsrc)
        for n, v in have.items():
            if n not in used and n.startswith(self.prefix):
                self._avail.setdefault(n[len(self.prefix):], v)     # shown so that check_specs can call it unexpected

    @staticmethod
    def _find_prefix(specs, have) -> str:
        if any(n in have for n in specs):
            return ""
        first = next(iter(specs), None)
        if first is None:
            return ""
        found = {n[:-len(first)] for n in have if n.endswith(first) and len(n) > len(first)}
        good = [p for p in found if sum(1 for n in specs if p + n in have) * 2 >= len(specs)]
        return sorted(good, key=len)[0] if good else ""

    @staticmethod
    def _fused_source(name: str):
        for part, half in (("gate_proj", 0), ("up_proj", 1)):
            head, sep, tail = name.rpartition(part)
            if sep and not head.endswith("gate_"):
                return head + "gate_up_proj" + tail, half
        return None

    @staticmethod
    def _fused_sibling(name: str):
        """The fused gate|up tensor that a stacked ``down_proj`` would be stored beside."""
        head, sep, tail = name.rpartition("down_proj")
        return head + "gate_up_proj" + tail if sep and not tail else None

    @staticmethod
    def _split_plan(shape, want, stacked_in_out: bool):
        """(axis to split, transpose afterwards) for a fused tensor of `shape` giving `want`, or
        None.  `stacked_in_out`: the name says [.., in, 2 * out]; otherwise it says [.., 2 * out, in]."""
        if len(shape) != len(want) or len(shape) < 2 or shape[:-2] != want[:-2]:
            return None
        rows = shape[-2:] == (2 * want[-2], want[-1])          # [.., 2 * out, in]
        cols = shape[-2:] == (want[-1], 2 * want[-2])          # [.., in, 2 * out]
        if rows and cols:
            cols, rows = stacked_in_out, not stacked_in_out
        if cols:
            return (len(shape) - 1, True)
        if rows:
            return (len(shape) - 2, False)
        return None

    def available(self):
        return dict(self._avail)

    def get(self, name: str) -> torch.Tensor:
        plan = self._plan[name]
        if plan[0] == "plain":
            return self.inner.get(plan[1])
        if plan[0] == "transpose":
            return self.inner.get(plan[1]).transpose(1, 2).contiguous()
        _, src, half, (axis, transpose) = plan
        t = self.inner.get(src)
        n = t.shape[axis] // 2
        t = t.narrow(axis, half * n, n)
        return (t.transpose(-1, -2) if transpose else t).contiguous()


class RandomSource(TensorSource):
    """Seeded random tensors: matrices N(0, std), norm weights U(0.9, 1.1).

    Every element is a function of (seed, tensor name, element index) alone (see
    weights/random_fill.py), so the values depend neither on the order of the requests nor on
    where they are made: with ``generate_on_device`` the tensors are filled straight into device
    memory by a kernel, otherwise on the host, and both give the same bits.  ``stored_dtype`` is
    what a file written from this source holds (values are rounded to it first);
    ``float32_names`` keeps tensors whose name ends with one of the given suffixes in float32."""

    def __init__(self, specs: Dict[str, ParamSpec], seed: int, compute_dtype: torch.dtype, device,
                 stored_dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                 float32_names: Iterable[str] = (), std_by_suffix: Optional[Dict[str, float]] = None,
                 generate_on_device: bool = False):
        self.specs = dict(specs)
        self.seed = int(seed)
        self.compute_dtype = compute_dtype
        self.device = torch.device(device)
        self.stored_dtype = stored_dtype
        self.std = float(std)
        self.float32_names = tuple(float32_names)
        self.std_by_suffix = dict(std_by_suffix or {})
        self.generate_on_device = generate_on_device and self.device.type == "cuda"
        self.where = f"random(seed={seed})"

    def stored_dtype_of(self, name: str) -> torch.dtype:
        spec = self.specs[name]
        if spec.kind == "int":
            return torch.int32
        if any(name.endswith(s) for s in self.float32_names):
            return torch.float32
        return self.stored_dtype

    def available(self):
        return {n: (s.shape, self.stored_dtype_of(n)) for n, s in self.specs.items()}

    def stored(self, name: str) -> torch.Tensor:
        """The tensor as a file would hold it (host unless generating on the device)."""
        from . import random_fill as rf

        spec = self.specs[name]
        key = rf.name_key(self.seed, name)
        sd = self.stored_dtype_of(name)
        kind = rf.FILL_INT if spec.kind == "int" else rf.FILL_UNIFORM if spec.init == INIT_NORM_WEIGHT else rf.FILL_NORMAL
        if self.generate_on_device:
            from .. import ops

            return ops.random_fill(torch.empty(spec.shape, dtype=sd, device=self.device), key, kind, self._std_of(name))
        return rf.host_tensor(spec.shape, key, kind, sd, self._std_of(name))

    def _std_of(self, name: str) -> float:
        for suffix, s in self.std_by_suffix.items():
            if name.endswith(suffix):
                return float(s)
        return self.std

    def get(self, name: str) -> torch.Tensor:
        t = self.stored(name)
        want = storage_dtype(t.dtype, self.compute_dtype)
        if t.dtype != want:
            t = t.to(want)
        return t.to(self.device)


# ---------------------------------------------------------------------------
def load_model_weights(model, source: TensorSource) -> None:
    """Check the source against the model's request, then let the parts take their tensors."""
    specs = model.param_specs()
    if isinstance(source, SafetensorsSource):
        source = LayoutAdapter(source, specs)        # other layouts of the same tensors (prefix, fused experts)
    check_specs(specs, source.available(), source.where)
    model.load_weights(source)


def write_random_model(config, out_dir: str, seed: int, stored_dtype: torch.dtype = torch.bfloat16,
                       std: float = 0.02, float32_names: Iterable[str] = (),
                       std_by_suffix: Optional[Dict[str, float]] = None) -> str:
    """Random-weights mode: a model folder (config.json, model.safetensors) from a
    configuration and a seed."""
    from ..config.base import save_config
    from ..registry import build_model

    model = build_model(config)
    specs = model.param_specs()
    # the values are a function of (seed, name, element) wherever they are made: on a machine with a
    # GPU the fill kernel makes them (a large model's file is then written in seconds, not minutes)
    on_gpu = torch.cuda.is_available()
    src = RandomSource(specs, seed, torch.float32, "cuda" if on_gpu else "cpu", stored_dtype=stored_dtype, std=std,
                       float32_names=float32_names, std_by_suffix=std_by_suffix, generate_on_device=on_gpu)
    os.makedirs(out_dir, exist_ok=True)
    save_config(config, out_dir)
    st.write_file(os.path.join(out_dir, "model.safetensors"), ((n, src.stored(n).cpu()) for n in sorted(specs)),
                  metadata={"format": "pt", "seed": str(seed)})
    return out_dir
