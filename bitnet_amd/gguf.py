"""GGUF container <-> the int8 x int2 decoder's state dict.

The CPU stack of the reference keeps a model as one GGUF file whose ternary
tensors are of type I2_S (written by utils/convert-hf-to-gguf-bitnet.py:666-727
and utils/convert-bitnet-embedding-to-gguf.py:428-492; consumed by
src/ggml-bitnet-mad.cpp:81-96).  This module reads such a file without any
third-party package (the reference relies on llama.cpp's gguf-py, which it does
not vendor), turns its tensors into what `decoder.Transformer` loads -- fused
wqkv / w13 in the GPU layout with four-slot scales, q/k rows in the decoder's
rotary order -- and writes the inverse.

Container layout (GGUF version 2 and 3, little endian):
  u32 magic "GGUF" | u32 version | u64 n_tensors | u64 n_kv
  n_kv  x (string key, u32 value type, value)
  n_tensors x (string name, u32 n_dims, u64 dims[n_dims] innermost first,
               u32 ggml type, u64 offset into the data section)
  padding to `general.alignment` (32 when absent) | tensor data, each tensor
  aligned likewise.  A string is u64 length + bytes, an array u32 element
  type + u64 count + elements.

An I2_S tensor of n x k elements occupies n*k/4 code bytes followed by 32
bytes that start with its fp32 scale (the layout `i2s.py` transcodes).

Not pinned by any file of the reference: the numeric id of the I2_S tensor
type (it is defined in the un-vendored llama.cpp fork; `I2_S_TYPE` below is
that fork's value and every function takes another) and the tensor names of
the `bitnet-b1.58` architecture (gguf-py's name map).  The reference does pin
the file type 40 of such a file (convert-hf-to-gguf-bitnet.py:158-159), the
per-tensor byte layout, that norms and one-dimensional tensors stay fp32 and
that q/k rows are stored in Hugging Face order (its BitnetModel,
convert-hf-to-gguf-bitnet.py:1031-1072, does not permute them).
"""
import mmap
import os
import struct
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import i2s
from .checkpoint import rope_rows_hf_to_interleaved
from .decoder import ModelArgs

GGUF_MAGIC = 0x46554747  # b"GGUF" read as a little-endian u32
DEFAULT_ALIGNMENT = 32
I2_S_TYPE = 36  # GGML_TYPE_I2_S of the reference's llama.cpp fork
FTYPE_MOSTLY_I2_S = 40  # convert-hf-to-gguf-bitnet.py:159

# ggml tensor types this reader decodes: id -> (numpy dtype, bytes per element)
_PLAIN_TYPES = {0: (np.float32, 4), 1: (np.float16, 2), 24: (np.int8, 1), 25: (np.int16, 2), 26: (np.int32, 4),
                27: (np.int64, 8), 28: (np.float64, 8), 30: (np.uint16, 2)}  # 30 = bf16, kept as raw bits
BF16_TYPE = 30

# metadata value types
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_T_STRING, _T_ARRAY = 8, 9


class GGUFError(ValueError):
    pass


class TensorInfo:
    __slots__ = ("name", "shape", "ggml_type", "offset", "nbytes")

    def __init__(self, name: str, shape: Tuple[int, ...], ggml_type: int, offset: int, nbytes: int):
        self.name, self.shape, self.ggml_type, self.offset, self.nbytes = name, shape, ggml_type, offset, nbytes

    def __repr__(self):
        return f"TensorInfo({self.name!r}, shape={self.shape}, type={self.ggml_type}, offset={self.offset}, nbytes={self.nbytes})"


def _tensor_nbytes(shape: Sequence[int], ggml_type: int, i2s_type: int) -> Optional[int]:
    n = 1
    for d in shape:
        n *= d
    if ggml_type == i2s_type:
        return n // 4 + i2s.I2S_TAIL_BYTES
    if ggml_type in _PLAIN_TYPES:
        return n * _PLAIN_TYPES[ggml_type][1]
    return None  # a block-quantised type this reader does not decode: sized by its neighbours


class GGUFReader:
    """Memory-maps a GGUF file; metadata in `.kv`, tensor directory in `.tensors`
    (shape in row-major order, i.e. the file's dims reversed)."""

    def __init__(self, path: str, i2s_type: int = I2_S_TYPE):
        self.path = path
        self.i2s_type = i2s_type
        self._f = open(path, "rb")
        size = os.fstat(self._f.fileno()).st_size
        if size < 24:
            self._f.close()
            raise GGUFError(f"{path}: {size} bytes is too short for a GGUF header")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        try:
            self._parse(size)
        except Exception:
            self.close()  # a refused file leaves no mapping or descriptor behind
            raise

    def _parse(self, size: int) -> None:
        path, i2s_type = self.path, self.i2s_type
        self._pos = 0
        magic, self.version = self._unpack("<II")
        if magic != GGUF_MAGIC:
            raise GGUFError(f"{path}: magic {magic:#x} is not GGUF")
        if self.version not in (2, 3):
            raise GGUFError(f"{path}: GGUF version {self.version} (2 and 3 are read)")
        n_tensors, n_kv = self._unpack("<QQ")
        self.kv: Dict[str, object] = {}
        for _ in range(n_kv):
            key = self._string()
            (vtype,) = self._unpack("<I")
            self.kv[key] = self._value(vtype)
        self.alignment = int(self.kv.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"{path}: alignment {self.alignment} is not a power of two")
        infos: List[Tuple[str, Tuple[int, ...], int, int]] = []
        for _ in range(n_tensors):
            name = self._string()
            (n_dims,) = self._unpack("<I")
            if n_dims > 8:
                raise GGUFError(f"{path}: tensor {name!r} with {n_dims} dimensions")
            dims = self._unpack("<%dQ" % n_dims) if n_dims else ()
            ggml_type, offset = self._unpack("<IQ")
            infos.append((name, tuple(reversed(dims)), ggml_type, offset))
        self.data_start = -(-self._pos // self.alignment) * self.alignment
        data_len = size - self.data_start
        order = sorted(range(len(infos)), key=lambda i: infos[i][3])
        self.tensors: Dict[str, TensorInfo] = {}
        for rank, i in enumerate(order):
            name, shape, ggml_type, offset = infos[i]
            if offset % self.alignment:
                raise GGUFError(f"{path}: tensor {name!r} at offset {offset}, not a multiple of {self.alignment}")
            nbytes = _tensor_nbytes(shape, ggml_type, i2s_type)
            upper = infos[order[rank + 1]][3] if rank + 1 < len(order) else data_len
            if nbytes is None:
                nbytes = upper - offset
            if nbytes < 0 or offset + nbytes > min(upper, data_len):
                raise GGUFError(f"{path}: tensor {name!r} ({nbytes} bytes at {offset}) runs past its place in the file")
            if name in self.tensors:
                raise GGUFError(f"{path}: tensor name {name!r} twice")
            self.tensors[name] = TensorInfo(name, shape, ggml_type, offset, nbytes)

    # -- parsing helpers ----------------------------------------------------
    def _unpack(self, fmt: str):
        try:
            n = struct.calcsize(fmt)
        except struct.error:  # a count field far beyond any file
            raise GGUFError(f"{self.path}: field count at byte {self._pos} is not credible") from None
        if self._pos + n > len(self._mm):
            raise GGUFError(f"{self.path}: truncated at byte {self._pos}")
        out = struct.unpack_from(fmt, self._mm, self._pos)
        self._pos += n
        return out

    def _string(self) -> str:
        (n,) = self._unpack("<Q")
        if self._pos + n > len(self._mm):
            raise GGUFError(f"{self.path}: string of {n} bytes at {self._pos} runs past the end")
        s = bytes(self._mm[self._pos : self._pos + n]).decode("utf-8", errors="replace")
        self._pos += n
        return s

    def _value(self, vtype: int):
        if vtype in _SCALARS:
            return self._unpack(_SCALARS[vtype])[0]
        if vtype == _T_STRING:
            return self._string()
        if vtype == _T_ARRAY:
            etype, count = self._unpack("<IQ")
            if etype in _SCALARS:
                fmt = _SCALARS[etype][1]
                return list(self._unpack("<%d%s" % (count, fmt))) if count else []
            if etype == _T_STRING:
                return [self._string() for _ in range(count)]
            raise GGUFError(f"{self.path}: array of value type {etype}")
        raise GGUFError(f"{self.path}: metadata value type {vtype}")

    # -- tensors --------------------------------------------------------------
    def raw(self, name: str) -> np.ndarray:
        """The tensor's bytes as stored (a view of the mapping, not a copy)."""
        t = self.tensors[name]
        return np.frombuffer(self._mm, dtype=np.uint8, count=t.nbytes, offset=self.data_start + t.offset)

    def plain(self, name: str) -> torch.Tensor:
        """An F32 / F16 / BF16 / integer tensor as a torch tensor of its shape (copied out of the mapping)."""
        t = self.tensors[name]
        if t.ggml_type not in _PLAIN_TYPES:
            raise GGUFError(f"tensor {name!r} has ggml type {t.ggml_type}, which is not a plain array")
        arr = self.raw(name).view(_PLAIN_TYPES[t.ggml_type][0]).reshape(t.shape).copy()
        if t.ggml_type == BF16_TYPE:
            return torch.from_numpy(arr.view(np.int16)).view(torch.bfloat16)
        return torch.from_numpy(arr)

    def i2s(self, name: str) -> Tuple[torch.Tensor, float, int, int]:
        """An I2_S tensor: (code bytes [n*k/4], scale, n, k)."""
        t = self.tensors[name]
        if t.ggml_type != self.i2s_type:
            raise GGUFError(f"tensor {name!r} has ggml type {t.ggml_type}, not I2_S ({self.i2s_type})")
        if len(t.shape) != 2:
            raise GGUFError(f"I2_S tensor {name!r} with shape {t.shape}: two dimensions expected")
        n, k = t.shape
        codes, scale = i2s.split_i2s_tensor(torch.from_numpy(self.raw(name).copy()), n, k)
        return codes, scale, n, k

    def close(self):
        self._mm.close()
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


# ---------------------------------------------------------------------------
# writing
# ---------------------------------------------------------------------------
def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    """Python value -> (type, payload): bool, int (i32 / u32 / i64 / u64 by range), float (f32), str, or a
    homogeneous list of those; a (type id, value) tuple forces a scalar type."""
    if isinstance(v, tuple):
        vtype, val = v
        return struct.pack("<I", vtype) + struct.pack(_SCALARS[vtype], val)
    if isinstance(v, bool):
        return struct.pack("<I?", 7, v)
    if isinstance(v, int):
        if 0 <= v < 2 ** 32:
            return struct.pack("<II", 4, v)
        if -(2 ** 31) <= v < 0:
            return struct.pack("<Ii", 5, v)
        return struct.pack("<IQ", 10, v) if v >= 0 else struct.pack("<Iq", 11, v)
    if isinstance(v, float):
        return struct.pack("<If", 6, v)
    if isinstance(v, str):
        return struct.pack("<I", _T_STRING) + _pack_string(v)
    if isinstance(v, (list, tuple)):
        if not v:
            return struct.pack("<IIQ", _T_ARRAY, 4, 0)
        first = _pack_value(v[0])
        etype = struct.unpack_from("<I", first)[0]
        body = b"".join(_pack_value(e)[4:] for e in v)
        return struct.pack("<IIQ", _T_ARRAY, etype, len(v)) + body
    raise GGUFError(f"metadata value {v!r} has no GGUF type")


def _tensor_payload(t, i2s_type: int) -> Tuple[Tuple[int, ...], int, bytes]:
    """(shape, ggml type, bytes) of one tensor to write: a torch tensor (fp32, fp16, bf16) or an
    (I2_S code bytes, scale, n, k) tuple."""
    if isinstance(t, tuple):
        codes, scale, n, k = t
        return (n, k), i2s_type, i2s.join_i2s_tensor(codes.reshape(-1).cpu(), float(scale)).numpy().tobytes()
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return tuple(t.shape), 0, t.numpy().tobytes()
    if t.dtype == torch.float16:
        return tuple(t.shape), 1, t.numpy().tobytes()
    if t.dtype == torch.bfloat16:
        return tuple(t.shape), BF16_TYPE, t.view(torch.int16).numpy().tobytes()
    raise GGUFError(f"tensor of dtype {t.dtype} cannot be written")


def write_gguf(path: str, kv: Dict[str, object], tensors: Dict[str, object], alignment: int = DEFAULT_ALIGNMENT,
               i2s_type: int = I2_S_TYPE) -> None:
    """A GGUF version 3 file with the given metadata and tensors (see `_tensor_payload`), in the order given."""
    kv = dict(kv)
    if alignment != DEFAULT_ALIGNMENT:
        kv["general.alignment"] = alignment
    head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(kv))
    for key, v in kv.items():
        head += _pack_string(key) + _pack_value(v)
    infos, offset, payloads = b"", 0, []
    for name, t in tensors.items():
        shape, ggml_type, data = _tensor_payload(t, i2s_type)
        infos += _pack_string(name) + struct.pack("<I", len(shape)) + struct.pack("<%dQ" % len(shape), *reversed(shape))
        infos += struct.pack("<IQ", ggml_type, offset)
        pad = -len(data) % alignment
        payloads.append(data + b"\0" * pad)
        offset += len(data) + pad
    with open(path, "wb") as f:
        f.write(head + infos)
        f.write(b"\0" * (-(len(head) + len(infos)) % alignment))
        for p in payloads:
            f.write(p)


# ---------------------------------------------------------------------------
# model level
# ---------------------------------------------------------------------------
def model_args_from_gguf(r: GGUFReader) -> ModelArgs:
    """ModelArgs from the `<architecture>.*` keys llama.cpp-style converters write."""
    arch = r.kv.get("general.architecture")
    if not isinstance(arch, str):
        raise GGUFError("general.architecture is missing")

    def get(key, default=None):
        v = r.kv.get(f"{arch}.{key}", default)
        if v is None:
            raise GGUFError(f"{arch}.{key} is missing")
        return v

    def f32(v):  # the double whose shortest decimal form the stored fp32 value has (1e-5, not 9.99999975e-06)
        return float(str(np.float32(v)))

    n_heads = int(get("attention.head_count"))
    vocab = r.kv.get(f"{arch}.vocab_size")
    if vocab is None:
        vocab = r.tensors["token_embd.weight"].shape[0]
    return ModelArgs(dim=int(get("embedding_length")), n_layers=int(get("block_count")), n_heads=n_heads,
                     n_kv_heads=int(get("attention.head_count_kv", n_heads)), vocab_size=int(vocab),
                     ffn_dim=int(get("feed_forward_length")), norm_eps=f32(get("attention.layer_norm_rms_epsilon", 1e-5)),
                     rope_theta=f32(get("rope.freq_base", 500000.0)))


def rope_rows_interleaved_to_hf(w: torch.Tensor, n_heads: int) -> torch.Tensor:
    """Inverse of checkpoint.rope_rows_hf_to_interleaved."""
    rows, cols = w.shape
    if rows % (2 * n_heads):
        raise ValueError(f"{rows} rows do not split into {n_heads} heads of pairs")
    d = rows // (2 * n_heads)
    return w.reshape(n_heads, d, 2, cols).transpose(1, 2).reshape(rows, cols)


def _fuse(r: GGUFReader, names: Iterable[str], heads: Sequence[Optional[int]], k_want: int, layout: str = "x86"):
    """I2_S tensors `names` (q/k with their head count for the rotary row order, None otherwise) ->
    (packed [N, k/4] int8, weight_scale bf16 [4])."""
    parts = []
    for name, h in zip(names, heads):
        codes, scale, n, k = r.i2s(name)
        if k != k_want:
            raise GGUFError(f"{name}: {k} columns, {k_want} expected")
        if h is not None:
            w = rope_rows_hf_to_interleaved(i2s.i2s_unpack(codes, n, k, layout), h).contiguous()
            codes = i2s.i2s_pack(w, layout)
        parts.append((codes, scale, n))
    return i2s.i2s_to_int2(parts, k_want, layout)


def gguf_to_int2_state(r: GGUFReader, args: Optional[ModelArgs] = None, dtype=torch.bfloat16,
                       layout: str = "x86") -> Dict[str, torch.Tensor]:
    """The state dict `decoder.Transformer(args)` loads, from a GGUF file of the
    bitnet-b1.58 architecture whose seven projections per block are I2_S tensors.  Embedding and norms
    are cast to `dtype`; `output.weight` is the file's own when it has one, else the embedding (tied,
    as gpu/convert_safetensors.py:88-91 does).  `layout` names the I2_S byte layout of the build that
    wrote the file (`i2s.I2S_LAYOUTS`; the file itself does not record it)."""
    a = args or model_args_from_gguf(r)
    st: Dict[str, torch.Tensor] = {}
    for layer in range(a.n_layers):
        b, p = f"blk.{layer}.", f"layers.{layer}."
        packed, scale = _fuse(r, [b + "attn_q.weight", b + "attn_k.weight", b + "attn_v.weight"], [a.n_heads, a.n_kv_heads, None], a.dim, layout)
        st[p + "attention.wqkv.weight"], st[p + "attention.wqkv.weight_scale"] = packed, scale
        packed, scale = _fuse(r, [b + "attn_output.weight"], [None], a.dim, layout)
        st[p + "attention.wo.weight"], st[p + "attention.wo.weight_scale"] = packed, scale
        packed, scale = _fuse(r, [b + "ffn_gate.weight", b + "ffn_up.weight"], [None, None], a.dim, layout)
        st[p + "feed_forward.w13.weight"], st[p + "feed_forward.w13.weight_scale"] = packed, scale
        packed, scale = _fuse(r, [b + "ffn_down.weight"], [None], a.ffn_dim, layout)
        st[p + "feed_forward.w2.weight"], st[p + "feed_forward.w2.weight_scale"] = packed, scale
        st[p + "attention_norm.weight"] = r.plain(b + "attn_norm.weight").to(dtype)
        st[p + "ffn_norm.weight"] = r.plain(b + "ffn_norm.weight").to(dtype)
        st[p + "attention.attn_sub_norm.weight"] = r.plain(b + "attn_sub_norm.weight").to(dtype)
        st[p + "feed_forward.ffn_sub_norm.weight"] = r.plain(b + "ffn_sub_norm.weight").to(dtype)
    st["tok_embeddings.weight"] = r.plain("token_embd.weight").to(dtype)
    st["output.weight"] = r.plain("output.weight").to(dtype) if "output.weight" in r.tensors else st["tok_embeddings.weight"]
    st["norm.weight"] = r.plain("output_norm.weight").to(dtype)
    return st


def int2_state_to_gguf(state: Dict[str, torch.Tensor], args: ModelArgs, path: str, name: str = "bitnet-amd export",
                       embed_dtype=torch.float16, i2s_type: int = I2_S_TYPE, layout: str = "x86") -> None:
    """The inverse: a packed decoder state dict -> a GGUF file with I2_S projections (q/k rows back in
    Hugging Face order), fp32 norms and an fp16 embedding, as the reference's converter lays a model
    out (convert-hf-to-gguf-bitnet.py:1120-1190).  No tokenizer metadata is written."""
    a = args
    hd = a.dim // a.n_heads
    arch = "bitnet-b1.58"
    kv = {"general.architecture": arch, "general.name": name, "general.file_type": FTYPE_MOSTLY_I2_S,
          f"{arch}.vocab_size": a.vocab_size, f"{arch}.embedding_length": a.dim, f"{arch}.block_count": a.n_layers,
          f"{arch}.feed_forward_length": a.ffn_dim, f"{arch}.attention.head_count": a.n_heads,
          f"{arch}.attention.head_count_kv": a.n_kv_heads, f"{arch}.rope.dimension_count": hd,
          f"{arch}.rope.freq_base": float(a.rope_theta), f"{arch}.attention.layer_norm_rms_epsilon": float(a.norm_eps)}
    tensors: Dict[str, object] = {"token_embd.weight": state["tok_embeddings.weight"].to(embed_dtype)}
    if not torch.equal(state["output.weight"], state["tok_embeddings.weight"]):
        tensors["output.weight"] = state["output.weight"].to(embed_dtype)
    tensors["output_norm.weight"] = state["norm.weight"].float()

    def parts(key, rows, heads):
        out = []
        for (codes, scale), n, h in zip(i2s.int2_to_i2s(state[key].cpu(), state[key.replace("weight", "weight_scale")].cpu(), rows, layout), rows, heads):
            k = state[key].shape[1] * 4
            if h is not None:
                codes = i2s.i2s_pack(rope_rows_interleaved_to_hf(i2s.i2s_unpack(codes, n, k, layout), h).contiguous(), layout)
            out.append((codes, scale, n, k))
        return out

    for layer in range(a.n_layers):
        b, p = f"blk.{layer}.", f"layers.{layer}."
        tensors[b + "attn_norm.weight"] = state[p + "attention_norm.weight"].float()
        q, k_, v = parts(p + "attention.wqkv.weight", [a.n_heads * hd, a.n_kv_heads * hd, a.n_kv_heads * hd], [a.n_heads, a.n_kv_heads, None])
        tensors[b + "attn_q.weight"], tensors[b + "attn_k.weight"], tensors[b + "attn_v.weight"] = q, k_, v
        tensors[b + "attn_sub_norm.weight"] = state[p + "attention.attn_sub_norm.weight"].float()
        (tensors[b + "attn_output.weight"],) = parts(p + "attention.wo.weight", [a.dim], [None])
        tensors[b + "ffn_norm.weight"] = state[p + "ffn_norm.weight"].float()
        g, u = parts(p + "feed_forward.w13.weight", [a.ffn_dim, a.ffn_dim], [None, None])
        tensors[b + "ffn_gate.weight"], tensors[b + "ffn_up.weight"] = g, u
        tensors[b + "ffn_sub_norm.weight"] = state[p + "feed_forward.ffn_sub_norm.weight"].float()
        (tensors[b + "ffn_down.weight"],) = parts(p + "feed_forward.w2.weight", [a.dim], [None])
    write_gguf(path, kv, tensors, i2s_type=i2s_type)
