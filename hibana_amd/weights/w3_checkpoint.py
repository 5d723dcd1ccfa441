"""The calibrated 3-bit checkpoint format (hibana/weights/w3_checkpoint.py:25-139 of the reference): a directory with
`manifest.json` (format 1, the target revision, per weight: file, sha256, shape, codebook) and one safetensors file per
matrix holding `planes` uint32 [N/32, K/128, 3, 32, 4], `scales` uint8 [N/32, K/128, 4, 32] and `row_scale` float32 [N]
in the reference's fragment order. Files are tensor-only and read with safetensors after their checksum matches.

Loading is where the gfx950 block layout is made: with `tile=True` (the default on a GPU device) a loaded matrix is
repacked once by `w3.tile(..., release=True)` and the fragment-order tensors are dropped, so a served model holds one
copy of each matrix.

Downloading published checkpoints (`fetch` in the reference) is not part of this module.
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch
from safetensors.torch import load as load_bytes, save_file

FORMAT_VERSION = 1


class Shard:
    """Which part of a checkpoint matrix a loader keeps (hibana/weights/sharding.py:31-44): `rows` cuts dim 0, whose
    entries are `unit` output rows each, `cols` the input dimension along `dim`. The base class keeps everything."""

    def rows(self, t: torch.Tensor, unit: int = 1) -> torch.Tensor:
        return t

    def cols(self, t: torch.Tensor, dim: int = -1) -> torch.Tensor:
        return t


REPLICATED = Shard()


class ExpertRange(Shard):
    """Experts lo .. hi - 1 of a stack of whole experts, `rows_per_expert` output rows each (the part one GPU keeps
    under expert parallelism, hibana/weights/sharding.py:81-96)."""

    def __init__(self, lo: int, hi: int, rows_per_expert: int):
        self.lo, self.hi, self.rows_per_expert = lo, hi, rows_per_expert

    def rows(self, t: torch.Tensor, unit: int = 1) -> torch.Tensor:
        if self.rows_per_expert % unit:
            raise ValueError("an expert's rows do not fill the tensor's row unit")
        per = self.rows_per_expert // unit
        return t[self.lo * per:self.hi * per]


def sha256(path: Path) -> str:
    digest = hashlib.sha256()
    with Path(path).open("rb") as handle:
        for block in iter(lambda: handle.read(8 * 2 ** 20), b""):
            digest.update(block)
    return digest.hexdigest()


def save_weight(path: Path, weight) -> dict:
    """Write one W3Weight (its fragment-order tensors) and return its manifest entry
    (hibana/weights/w3_checkpoint.py:47-54)."""
    if weight.planes is None or weight.scales is None:
        raise ValueError("the fragment-order tensors were released; a tiled-only weight cannot be saved")
    path = Path(path)
    path.parent.mkdir(parents=True, exist_ok=True)
    temporary = path.with_suffix(".tmp")
    save_file({"planes": weight.planes.cpu().contiguous(), "scales": weight.scales.cpu().contiguous(),
               "row_scale": weight.row_scale.cpu().contiguous()}, str(temporary))
    temporary.replace(path)
    return {"file": path.name, "sha256": sha256(path), "out_features": weight.out_features, "in_features": weight.in_features,
            "codebook": list(weight.codebook)}


class CalibratedWeights:
    def __init__(self, directory: str | Path, revision: str):
        """The calibrated copies in `directory` for the target at `revision` (hibana/weights/w3_checkpoint.py:57-65)."""
        self.directory = Path(directory)
        self.manifest = json.loads((self.directory / "manifest.json").read_text())
        if self.manifest.get("format") != FORMAT_VERSION or self.manifest.get("target_revision") != revision:
            raise ValueError("calibrated W3 checkpoint format or target revision does not match")
        self.weights = self.manifest["weights"]
        self.identity = sha256(self.directory / "manifest.json")

    def paths(self, names) -> list[tuple[Path, str]]:
        """The files of `names` and their recorded checksums."""
        return [(self.directory / self.weights[name]["file"], self.weights[name]["sha256"]) for name in names]

    @staticmethod
    def expert_names(layer: int) -> list[str]:
        return [f"layers.{layer}.experts.w13", f"layers.{layer}.experts.w2"]

    def expert_layers(self) -> set[int]:
        """The layers whose routed experts the checkpoint carries."""
        return {int(name.split(".")[1]) for name in self.weights if name.startswith("layers.") and ".experts." in name}

    def load(self, name: str, linear, shard: Shard = REPLICATED, tile: bool | None = None):
        """`linear`'s copy (its `out_features` x `in_features`, on `linear.weight.device`), in `linear`'s row order: an
        MLP's gate|up interleaved in blocks of `linear.pairs` (hibana/weights/w3_checkpoint.py:80-88)."""
        pairs = getattr(linear, "pairs", 0)
        weight = self._load(name, linear.out_features, linear.in_features, linear.weight.device, shard, tile=False)
        if pairs:
            from hibana_amd.kernels.w3 import interleave_rows
            weight = interleave_rows(weight, pairs)
        return self._finish(weight, tile)

    def load_many(self, items):
        """`load` for each (name, linear, shard) in order."""
        for name, linear, shard in items:
            yield self.load(name, linear, shard)

    def load_experts(self, layer: int, experts: int, inter: int, hidden: int, device, lo: int = 0, hi: int | None = None,
                     tile: bool | None = None):
        """Layer `layer`'s routed experts lo .. hi - 1 (all by default): fc1 (rows in w3_moe.fc1_order) and fc2 stacked
        over the experts (hibana/weights/w3_checkpoint.py:104-113)."""
        from hibana_amd.kernels import w3_moe
        hi = experts if hi is None else hi
        w13, w2 = self.expert_names(layer)
        fc1 = self._load(w13, (hi - lo) * 2 * inter, hidden, device, ExpertRange(lo, hi, 2 * inter), tile=False)
        fc2 = self._load(w2, (hi - lo) * hidden, inter, device, ExpertRange(lo, hi, hidden), tile=False)
        ex = w3_moe.W3Experts.from_stacked(fc1, fc2, hi - lo, base=lo)
        if self._wants_tile(tile, torch.device(device)):
            w3_moe.tile(ex, release=True)
        return ex

    @staticmethod
    def _wants_tile(tile: bool | None, device: torch.device) -> bool:
        return device.type == "cuda" if tile is None else tile

    def _finish(self, weight, tile: bool | None):
        if self._wants_tile(tile, weight.row_scale.device):
            from hibana_amd.kernels import w3
            w3.tile(weight, release=True)
        return weight

    def _load(self, name: str, out_features: int, in_features: int, device, shard: Shard = REPLICATED, tile: bool | None = None):
        from hibana_amd.kernels.w3 import W3Weight, _codebook, lut_of
        entry = self.weights[name]
        n, k = entry["out_features"], entry["in_features"]
        filename = entry["file"]
        if Path(filename).name != filename:
            raise ValueError("calibrated W3 files must be directly inside the checkpoint")
        data = (self.directory / filename).read_bytes()  # read once, checked before it is parsed
        if hashlib.sha256(data).hexdigest() != entry["sha256"]:
            raise ValueError(f"calibrated W3 checksum mismatch for {name}")
        tensors = load_bytes(data)
        expected = {"planes": ((n // 32, k // 128, 3, 32, 4), torch.uint32), "scales": ((n // 32, k // 128, 4, 32), torch.uint8),
                    "row_scale": ((n,), torch.float32)}
        if tensors.keys() != expected.keys() or any(tuple(tensors[key].shape) != shape or tensors[key].dtype != dtype
                                                     for key, (shape, dtype) in expected.items()):
            raise ValueError(f"invalid calibrated W3 tensors for {name}")
        levels = _codebook(entry["codebook"])
        # the fragment tensors index 32 rows by dim 0 and a 128-wide K chunk by dim 1; row scales follow the rows
        planes, scales = (shard.cols(shard.rows(tensors[key], 32), dim=1) for key in ("planes", "scales"))
        row_scale = shard.rows(tensors["row_scale"])
        n, k = row_scale.shape[0], planes.shape[1] * 128
        if (n, k) != (out_features, in_features):
            raise ValueError(f"calibrated W3 shape mismatch for {name}")
        weight = W3Weight(*(t.contiguous().to(device) for t in (planes, scales, row_scale)), n, k, levels, lut_of(levels))
        return self._finish(weight, tile)
