"""CNQ1 container reader: the tensor table and the bytes the NVFP4 load path needs.

Mirrors ``engine/src/cnq.rs`` of the reference for exactly that: ``read_index_trailer`` (:143-167),
``classify_index`` / ``parse_model_block`` (:175-239), ``parse_tensor_index`` (:715-733), ``Cnq::open_checked``
(:952-983), ``find`` (:1051-1062), ``byte_len`` (:1071-1078), ``read_bytes`` / ``read_range`` (:1122-1135).
Layout: magic ``CNQ1``, payload blob from ``blob_offset`` (12), the index JSON as a trailer followed by its
length as a u64 LE in the last 8 bytes; tensor offsets are relative to the blob start.  An NVFP4 tensor is
36 bytes per 64 values, rows contiguous, plus one f32 global scale in the index.

Same refusals, same texts: every reason ``open_checked`` returns as ``Err(String)`` is raised here as
``CnqRefused`` with that text; ``Cnq.open`` prefixes ``[cnq] refused: {path}: `` as the reference's panic does;
``find`` raises ``KeyError("tensor not found: {name} [{section}]")``.  Not mirrored (outside this path): the
overlay container, the file mapping, the page-cache advice and the PLE row fetch.
"""
from __future__ import annotations

import hashlib
import json
import os
import struct
from dataclasses import dataclass, field

import numpy as np

# sha256 of the index trailer of the one index-v1 container the reference accepts (cnq.rs:86) and its length (:89)
CNQ45M_INDEX_SHA256 = "a21afc43203d983e46be5dd378ac5fb34581ab31fb5a0f6e8093d4730078c4ba"
CNQ45M_INDEX_LEN = 473_528
V1_REFUSAL = "CNQ index v1 is only accepted for the Flash-Next CNQ4.5-M container of record"


class CnqRefused(ValueError):
    pass


@dataclass(frozen=True)
class TensorInfo:
    name: str
    section: str
    dtype: str
    offset: int  # relative to the blob start
    n_values: int
    global_scale: float
    shape: tuple = ()


@dataclass(frozen=True)
class ModelBlock:
    family: str
    model_type: str
    recipe: str
    config_json: str
    generation_config_json: str
    source_repo: str
    source_revision: str
    geo: object = None
    shards: object = None


def sha256_hex(b: bytes) -> str:
    return hashlib.sha256(b).hexdigest()


def read_index_trailer(path: str):
    """(file length, raw index bytes, parsed index) - magic and index length checked."""
    file_len = os.path.getsize(path)
    if file_len < 20:
        raise CnqRefused(f"{file_len} B is too small to be a CNQ1 container")
    with open(path, "rb") as f:
        magic = f.read(4)
        if magic != b"CNQ1":
            raise CnqRefused(f"magic is {list(magic)}, not CNQ1")
        f.seek(file_len - 8)
        idx_len = struct.unpack("<Q", f.read(8))[0]
        if idx_len == 0 or idx_len + 20 > file_len:
            raise CnqRefused(f"index length {idx_len} does not fit a {file_len} B file")
        f.seek(file_len - 8 - idx_len)
        ib = f.read(idx_len)
    try:
        index = json.loads(ib)
    except ValueError as e:
        raise CnqRefused(f"index json: {e}") from None
    return file_len, ib, index


def _req_str(v, what: str) -> str:
    if not isinstance(v, str):
        raise CnqRefused(f"CNQ index v2: `{what}` missing or not a string")
    return v


def parse_model_block(index: dict) -> ModelBlock:
    m = index.get("model")
    if not isinstance(m, dict):
        raise CnqRefused("CNQ index v2 without a `model` block")
    config_json = _req_str(m.get("config_json"), "model.config_json")
    generation_config_json = _req_str(m.get("generation_config_json"), "model.generation_config_json")
    for what, text in (("config_json", config_json), ("generation_config_json", generation_config_json)):
        want = _req_str(m.get(f"{what}_sha256"), f"model.{what}_sha256")
        got = sha256_hex(text.encode())
        if got != want:
            raise CnqRefused(f"CNQ index v2: model.{what} hashes to {got}, the index records {want} - the stored config was altered")
    src = m.get("source") if isinstance(m.get("source"), dict) else {}
    return ModelBlock(
        family=_req_str(m.get("family"), "model.family"),
        model_type=_req_str(m.get("model_type"), "model.model_type"),
        recipe=_req_str(index.get("recipe"), "recipe"),
        config_json=config_json,
        generation_config_json=generation_config_json,
        source_repo=_req_str(src.get("repo"), "model.source.repo"),
        source_revision=_req_str(src.get("revision"), "model.source.revision"),
        geo=m.get("geo"),
        shards=src.get("shards"),
    )


def classify_index(index_bytes: bytes, index: dict, v1_of_record: str = CNQ45M_INDEX_SHA256):
    """None for the v1 container of record, a ModelBlock for an index v2; anything else is refused."""
    fv = index.get("format_version")
    if fv is None:
        v = index.get("version")
        if v is not None and v != 1:
            raise CnqRefused(f"CNQ index `version` {json.dumps(v)} without a `format_version` - not an index this engine reads")
        got = sha256_hex(index_bytes)
        if got == v1_of_record:
            return None
        raise CnqRefused(
            f"{V1_REFUSAL} (index sha256 {got}, {len(index_bytes)} B; of record {v1_of_record}, {CNQ45M_INDEX_LEN} B) - "
            "re-convert the checkpoint: the converter writes index v2, which carries the model's config")
    if fv == 2 and not isinstance(fv, bool):
        return parse_model_block(index)
    raise CnqRefused(f"CNQ index format_version {json.dumps(fv)} is not one this engine reads (it reads 2, and v1 only for the container of record)")


def parse_tensor_index(index: dict) -> list:
    out = []
    for t in index.get("tensors") or []:
        gs = t.get("global_scale")
        out.append(TensorInfo(
            name=t["name"], section=t["section"], dtype=t["dtype"], offset=int(t["offset"]), n_values=int(t["n_values"]),
            global_scale=float(np.float32(gs if isinstance(gs, (int, float)) else 1.0)),
            shape=tuple(int(v) for v in (t.get("shape") or ()))))
    return out


@dataclass
class Cnq:
    path: str
    blob_offset: int
    tensors: list
    model_block: ModelBlock | None
    file_len: int
    _f: object = field(default=None, repr=False)

    @staticmethod
    def open_checked(path: str) -> "Cnq":
        file_len, ib, index = read_index_trailer(path)
        model = classify_index(ib, index)
        bo = index.get("blob_offset")
        if not isinstance(bo, int) or isinstance(bo, bool) or bo < 0:
            raise CnqRefused("index has no blob_offset")
        return Cnq(path, bo, parse_tensor_index(index), model, file_len, open(path, "rb"))

    @staticmethod
    def open(path: str) -> "Cnq":
        try:
            return Cnq.open_checked(path)
        except CnqRefused as why:
            raise CnqRefused(f"[cnq] refused: {path}: {why}") from None

    def close(self) -> None:
        if self._f is not None:
            self._f.close()
            self._f = None

    def model(self) -> ModelBlock | None:
        return self.model_block

    def family(self) -> str:
        return self.model_block.family if self.model_block else "FlashNext"

    def find(self, name: str, section: str) -> TensorInfo:
        for t in self.tensors:
            if t.name == name and t.section == section:
                return t
        raise KeyError(f"tensor not found: {name} [{section}]")

    @staticmethod
    def byte_len(t: TensorInfo) -> int:
        if t.dtype == "bf16":
            return t.n_values * 2
        if t.dtype == "i64":
            return t.n_values * 8
        if t.dtype == "f32":
            return t.n_values * 4
        return (t.n_values + 63) // 64 * 36  # nvfp4

    def _read_at(self, off: int, n: int) -> np.ndarray:
        if off < 0 or off + n > self.file_len - 8:
            raise CnqRefused(f"read of {n} B at {off} runs off the payload of a {self.file_len} B container")
        self._f.seek(off)
        raw = self._f.read(n)
        if len(raw) != n:
            raise IOError(f"{self.path}: short read ({len(raw)} of {n} B at {off})")
        return np.frombuffer(raw, np.uint8).copy()  # writable: callers hand it to torch

    def read_bytes(self, t: TensorInfo) -> np.ndarray:
        return self._read_at(self.blob_offset + t.offset, Cnq.byte_len(t))

    def read_range(self, t: TensorInfo, rel_off: int, n: int) -> np.ndarray:
        """A byte range of a tensor (row-aligned reads for expert slabs)."""
        return self._read_at(self.blob_offset + t.offset + rel_off, n)
