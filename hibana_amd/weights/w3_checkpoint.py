"""The calibrated 3-bit checkpoint format (hibana/weights/w3_checkpoint.py:25-139 of the reference): a directory with
`manifest.json` (format 1, the target revision, per weight: file, sha256, shape, codebook) and one safetensors file per
matrix holding `planes` uint32 [N/32, K/128, 3, 32, 4], `scales` uint8 [N/32, K/128, 4, 32] and `row_scale` float32 [N]
in the reference's fragment order. Files are tensor-only and read with safetensors after their checksum matches.

Loading is where the gfx950 block layout is made: with `tile=True` (the default on a GPU device) a loaded matrix is
repacked once by `w3.tile(..., release=True)` and the fragment-order tensors are dropped, so a served model holds one
copy of each matrix.

Reading goes through three small steps, each with one job: `ManifestEntry` (a manifest record, validated when it is
parsed), `read_verified` (bytes of a file whose digest matches) and `FragmentTensors` (the three tensors of a file,
checked against the shapes the record implies, then cut to a shard).

Downloading published checkpoints (`fetch` in the reference) is not part of this module.
"""
from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass
from pathlib import Path

import torch
from safetensors.torch import load as load_bytes, save_file

FORMAT_VERSION = 1
_READ_BLOCK = 8 << 20


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
    """Hex digest of a file, read in blocks."""
    state = hashlib.sha256()
    with open(path, "rb") as stream:
        while True:
            block = stream.read(_READ_BLOCK)
            if not block:
                return state.hexdigest()
            state.update(block)


def read_verified(path: Path, digest: str, what: str) -> bytes:
    """The file's bytes, read once and refused before anything parses them unless their SHA-256 is `digest`."""
    data = Path(path).read_bytes()
    if hashlib.sha256(data).hexdigest() != digest:
        raise ValueError(f"calibrated W3 checksum mismatch for {what}")
    return data


@dataclass(frozen=True)
class ManifestEntry:
    """One weight of the manifest: {"file", "sha256", "out_features", "in_features", "codebook"}."""
    name: str
    file: str
    sha256: str
    out_features: int
    in_features: int
    codebook: tuple[float, ...]

    @classmethod
    def parse(cls, name: str, record: dict) -> "ManifestEntry":
        file = str(record["file"])
        if Path(file).name != file:  # no directories, no "..": a manifest names files of its own folder only
            raise ValueError("calibrated W3 files must be directly inside the checkpoint")
        return cls(name, file, str(record["sha256"]), int(record["out_features"]), int(record["in_features"]),
                   tuple(float(v) for v in record["codebook"]))

    def record(self) -> dict:
        return {"file": self.file, "sha256": self.sha256, "out_features": self.out_features, "in_features": self.in_features,
                "codebook": list(self.codebook)}

    def tensor_spec(self) -> dict[str, tuple[tuple[int, ...], torch.dtype]]:
        """Name -> (shape, dtype) of the tensors the file must hold, and no others."""
        tiles, chunks = self.out_features // 32, self.in_features // 128
        return {"planes": ((tiles, chunks, 3, 32, 4), torch.uint32), "scales": ((tiles, chunks, 4, 32), torch.uint8),
                "row_scale": ((self.out_features,), torch.float32)}


@dataclass
class FragmentTensors:
    planes: torch.Tensor
    scales: torch.Tensor
    row_scale: torch.Tensor

    @classmethod
    def parse(cls, data: bytes, entry: ManifestEntry) -> "FragmentTensors":
        tensors = load_bytes(data)
        spec = entry.tensor_spec()
        ok = set(tensors) == set(spec) and all(tuple(tensors[k].shape) == shape and tensors[k].dtype == dtype for k, (shape, dtype) in spec.items())
        if not ok:
            raise ValueError(f"invalid calibrated W3 tensors for {entry.name}")
        return cls(tensors["planes"], tensors["scales"], tensors["row_scale"])

    def cut(self, shard: Shard) -> "FragmentTensors":
        """The shard's part: dim 0 of planes / scales counts 32-row tiles, dim 1 128-wide K chunks; row scales go with
        the rows."""
        return FragmentTensors(shard.cols(shard.rows(self.planes, 32), dim=1), shard.cols(shard.rows(self.scales, 32), dim=1),
                               shard.rows(self.row_scale))

    @property
    def shape(self) -> tuple[int, int]:
        return self.row_scale.shape[0], self.planes.shape[1] * 128


def save_weight(path: Path, weight) -> dict:
    """Write one W3Weight (its fragment-order tensors) and return its manifest entry
    (hibana/weights/w3_checkpoint.py:47-54). The file appears under its name only once it is complete."""
    if weight.planes is None or weight.scales is None:
        raise ValueError("the fragment-order tensors were released; a tiled-only weight cannot be saved")
    path = Path(path)
    path.parent.mkdir(parents=True, exist_ok=True)
    staging = path.with_suffix(".tmp")
    host = {key: getattr(weight, key).detach().cpu().contiguous() for key in ("planes", "scales", "row_scale")}
    save_file(host, str(staging))
    staging.replace(path)
    return ManifestEntry(path.stem, path.name, sha256(path), weight.out_features, weight.in_features, tuple(weight.codebook)).record()


class CalibratedWeights:
    def __init__(self, directory: str | Path, revision: str):
        """The calibrated copies in `directory` for the target at `revision` (hibana/weights/w3_checkpoint.py:57-65)."""
        self.directory = Path(directory)
        manifest_path = self.directory / "manifest.json"
        self.manifest = json.loads(manifest_path.read_text())
        found = (self.manifest.get("format"), self.manifest.get("target_revision"))
        if found != (FORMAT_VERSION, revision):
            raise ValueError("calibrated W3 checkpoint format or target revision does not match")
        self.weights = self.manifest["weights"]
        self.identity = sha256(manifest_path)

    def entry(self, name: str) -> ManifestEntry:
        return ManifestEntry.parse(name, self.weights[name])

    def paths(self, names) -> list[tuple[Path, str]]:
        """The files of `names` and their recorded checksums."""
        return [(self.directory / self.weights[n]["file"], self.weights[n]["sha256"]) for n in names]

    @staticmethod
    def expert_names(layer: int) -> list[str]:
        return [f"layers.{layer}.experts.{part}" for part in ("w13", "w2")]

    def expert_layers(self) -> set[int]:
        """The layers whose routed experts the checkpoint carries."""
        layers = set()
        for name in self.weights:
            parts = name.split(".")
            if len(parts) >= 4 and parts[0] == "layers" and parts[2] == "experts":
                layers.add(int(parts[1]))
        return layers

    def load(self, name: str, linear, shard: Shard = REPLICATED, tile: bool | None = None):
        """`linear`'s copy (its `out_features` x `in_features`, on `linear.weight.device`), in `linear`'s row order: an
        MLP's gate|up interleaved in blocks of `linear.pairs` (hibana/weights/w3_checkpoint.py:80-88)."""
        weight = self._load(name, linear.out_features, linear.in_features, linear.weight.device, shard, tile=False)
        block = getattr(linear, "pairs", 0)
        if block:
            from hibana_amd.kernels.w3 import interleave_rows
            weight = interleave_rows(weight, block)
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
        held = hi - lo
        stacks = []
        for name, rows, k in zip(self.expert_names(layer), (2 * inter, hidden), (hidden, inter)):
            stacks.append(self._load(name, held * rows, k, device, ExpertRange(lo, hi, rows), tile=False))
        ex = w3_moe.W3Experts.from_stacked(stacks[0], stacks[1], held, base=lo)
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
        from hibana_amd.kernels import w3
        entry = self.entry(name)
        data = read_verified(self.directory / entry.file, entry.sha256, name)
        part = FragmentTensors.parse(data, entry).cut(shard)
        if part.shape != (out_features, in_features):
            raise ValueError(f"calibrated W3 shape mismatch for {name}")
        levels = w3._codebook(entry.codebook)
        on_device = [t.contiguous().to(device) for t in (part.planes, part.scales, part.row_scale)]
        return self._finish(w3.W3Weight(*on_device, out_features, in_features, levels, w3.lut_of(levels)), tile)
