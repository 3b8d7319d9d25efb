"""GGUF v3 checkpoints: writer, reader, tensor serializers and the per-architecture tensor names.

Host-side mirror of the reference's checkpoint wire format, so that a run on this backend can start
from, and hand back to, the reference (and llama.cpp):

  * container: src/gguf/gguf.ts (GGUFWriter :127-277, readGGUF :416-454)
  * tensor bytes: src/gguf/quantize.ts (F32, F16, Q8_0, Q4_0 serializers :21-110, dequantize :154-223,
    BF16 read-only) and src/gguf/f16.ts (the float16 conversion, including its rounding of
    subnormal halves)
  * shared metadata block and loaders: src/arch/common.ts (startGGUF :96-114, addMatrix / addVector
    :32-49, tensorLoader :134-181, diffFields :196-214)
  * names, metadata keys and the llama Q/K row order: src/arch/llama.ts:104-129, 291-312, 372-445;
    src/arch/qwen3.ts:299-322, 359-420; src/arch/gemma3.ts:359-380, 424-489

Everything is little-endian and byte-exact; nothing here touches the GPU.
"""
from __future__ import annotations

import struct
import numpy as np

from .arch import LAYER_KEYS, Model, ModelConfig, param_names, param_shape

MAGIC = 0x46554747          # "GGUF"
VERSION = 3
DEFAULT_ALIGNMENT = 32

# gguf_metadata_value_type
UINT8, INT8, UINT16, INT16, UINT32, INT32, FLOAT32, BOOL, STRING, ARRAY, UINT64, INT64, FLOAT64 = range(13)

# ggml tensor types this format reads or writes
F32, F16, Q4_0, Q8_0, BF16 = 0, 1, 2, 8, 30
QK = 32                     # block size of Q4_0 and Q8_0
BLOCK_BYTES = {Q8_0: 2 + QK, Q4_0: 2 + QK // 2}
QUANT_NAMES = ("f32", "f16", "q8_0", "q4_0")
_GGML_TYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K",
                    11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 16: "IQ2_XXS", 17: "IQ2_XS", 19: "IQ3_XXS",
                    20: "IQ1_S", 21: "IQ4_NL", 23: "IQ3_S", 24: "IQ2_S", 26: "IQ4_XS", 30: "BF16"}


# ---- float16 (f16.ts) -------------------------------------------------------------------------------
def f32_to_f16_bits(values) -> np.ndarray:
    """float32 -> uint16 half bits, the reference's conversion (f16.ts:5-46): round-to-nearest-even for normal
    halves, round-half-up for subnormal halves, magnitudes below 2^-25 flushed to signed zero, NaN payloads
    reduced to one quiet bit."""
    x = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.int64)
    sign = (x >> 16) & 0x8000
    mant = x & 0x007FFFFF
    exp = (x >> 23) & 0xFF
    e = exp - 127 + 15
    out = np.zeros(x.shape, dtype=np.int64)
    # normal halves
    half = (e << 10) | (mant >> 13)
    round_bit = (mant >> 12) & 1
    sticky = (mant & 0x0FFF) != 0
    half = half + (((round_bit == 1) & (sticky | ((half & 1) == 1))).astype(np.int64))
    # subnormal halves: implicit leading one, shift, round half up
    m1 = mant | 0x00800000
    shift = np.clip(14 - e, 1, 62)
    sub = (m1 >> shift) + ((m1 >> (shift - 1)) & 1)
    out = np.where(e <= 0, np.where(e < -10, 0, sub), half)
    out = np.where(e >= 0x1F, 0x7C00, out)
    out = np.where(exp == 0xFF, 0x7C00 | np.where(mant != 0, 0x0200, 0), out)
    return (sign | out).astype(np.uint16)


def f16_bits_to_f32(bits) -> np.ndarray:
    """uint16 half bits -> float32 (f16.ts:49-77); exact, subnormals included."""
    return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


# ---- serializers (quantize.ts) ----------------------------------------------------------------------
def _js_round(x: np.ndarray) -> np.ndarray:
    """Math.round: halves go towards +infinity."""
    return np.floor(x + 0.5)


def serialize(data, quant: str):
    """(ggml type id, bytes) of a flat float32 array in the named format."""
    d = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
    if quant == "f32":
        return F32, d.astype("<f4").tobytes()
    if quant == "f16":
        return F16, f32_to_f16_bits(d).astype("<u2").tobytes()
    if quant not in ("q8_0", "q4_0"):
        raise ValueError(f'unknown quant "{quant}" (valid: {", ".join(QUANT_NAMES)})')
    if d.size % QK != 0:
        raise ValueError(f"{quant.upper()} needs a length multiple of {QK}, got {d.size}")
    blocks = d.reshape(-1, QK).astype(np.float64)
    nb = blocks.shape[0]
    if quant == "q8_0":
        # scale = max|x| / 127, q = round(x / scale) clamped to [-127, 127]; block = f16 scale + 32 int8
        amax = np.abs(blocks).max(axis=1)
        scale = amax / 127.0
        inv = np.where(scale != 0, 1.0 / np.where(scale != 0, scale, 1.0), 0.0)
        q = np.clip(_js_round(blocks * inv[:, None]), -127, 127).astype(np.int8)
        out = np.empty((nb, BLOCK_BYTES[Q8_0]), dtype=np.uint8)
        out[:, :2] = f32_to_f16_bits(scale.astype(np.float32)).astype("<u2").view(np.uint8).reshape(nb, 2)
        out[:, 2:] = q.view(np.uint8)
        return Q8_0, out.tobytes()
    # q4_0: the value of largest magnitude keeps its sign, scale = that / -8, nibble = floor(x / scale + 8.5) in
    # [0, 15]; byte j holds element j (low nibble) and element j + 16 (high nibble)
    idx = np.abs(blocks).argmax(axis=1)
    vmax = blocks[np.arange(nb), idx]
    scale = vmax / -8.0
    inv = np.where(scale != 0, 1.0 / np.where(scale != 0, scale, 1.0), 0.0)
    n = np.clip(np.floor(blocks * inv[:, None] + 8.5), 0, 15).astype(np.uint8)
    out = np.empty((nb, BLOCK_BYTES[Q4_0]), dtype=np.uint8)
    out[:, :2] = f32_to_f16_bits(scale.astype(np.float32)).astype("<u2").view(np.uint8).reshape(nb, 2)
    out[:, 2:] = n[:, :QK // 2] | (n[:, QK // 2:] << 4)
    return Q4_0, out.tobytes()


def bytes_for(ttype: int, count: int):
    """Bytes `count` elements of a ggml type occupy, or None for a type this reader cannot decode
    (quantize.ts:132-152)."""
    if ttype in BLOCK_BYTES:
        if count % QK != 0:
            raise ValueError(f"dequantize: ggml type {ttype} needs a count multiple of {QK}, got {count}")
        return count // QK * BLOCK_BYTES[ttype]
    if ttype == F32:
        return count * 4
    if ttype in (F16, BF16):
        return count * 2
    return None


def dequantize(ttype: int, data: bytes, count: int) -> np.ndarray:
    """Inverse of the serializers, plus BF16 (read only). The buffer may carry the file's alignment padding."""
    need = bytes_for(ttype, count)
    if need is not None and len(data) < need:
        raise ValueError(f"dequantize: {count} elements of ggml type {ttype} need {need} bytes, got {len(data)}")
    buf = np.frombuffer(data, dtype=np.uint8, count=need if need is not None else 0)
    if ttype == F32:
        return buf.view("<f4").astype(np.float32)
    if ttype == F16:
        return f16_bits_to_f32(buf.view("<u2"))
    if ttype == BF16:
        return (buf.view("<u2").astype(np.uint32) << 16).view(np.float32)
    if ttype == Q8_0:
        b = buf.reshape(-1, BLOCK_BYTES[Q8_0])
        d = f16_bits_to_f32(np.ascontiguousarray(b[:, :2]).view("<u2").reshape(-1))
        return (b[:, 2:].view(np.int8).astype(np.float32) * d[:, None]).reshape(-1)
    if ttype == Q4_0:
        b = buf.reshape(-1, BLOCK_BYTES[Q4_0])
        d = f16_bits_to_f32(np.ascontiguousarray(b[:, :2]).view("<u2").reshape(-1))
        lo = (b[:, 2:] & 0x0F).astype(np.float32) - 8.0
        hi = (b[:, 2:] >> 4).astype(np.float32) - 8.0
        return (np.concatenate([lo, hi], axis=1) * d[:, None]).reshape(-1)
    name = _GGML_TYPE_NAMES.get(ttype, f"id {ttype}")
    raise ValueError(f"Unsupported GGUF tensor type {name}. This reader dequantizes F32, F16, Q8_0, and Q4_0 only; "
                     "k-quants and other block formats are not supported. Load an F16/Q8_0/Q4_0 GGUF, or re-export "
                     "the source model at one of those types.")


# ---- container (gguf.ts) ----------------------------------------------------------------------------
def _gguf_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


class GGUFWriter:
    """Collects metadata key/values and tensors in call order; build() returns the whole file."""

    def __init__(self):
        self.meta: list = []          # (key, kind, value)
        self.tensors: list = []       # (name, dims in ggml order, type id, bytes)
        self.alignment = DEFAULT_ALIGNMENT

    def _add(self, key, kind, v):
        self.meta.append((key, kind, v))
        return self

    def meta_u32(self, key, v): return self._add(key, "u32", int(v))
    def meta_i32(self, key, v): return self._add(key, "i32", int(v))
    def meta_u64(self, key, v): return self._add(key, "u64", int(v))
    def meta_f32(self, key, v): return self._add(key, "f32", float(v))
    def meta_bool(self, key, v): return self._add(key, "bool", bool(v))
    def meta_string(self, key, v): return self._add(key, "string", str(v))
    def meta_arr_str(self, key, v): return self._add(key, "arr_str", list(v))
    def meta_arr_i32(self, key, v): return self._add(key, "arr_i32", list(v))
    def meta_arr_f32(self, key, v): return self._add(key, "arr_f32", list(v))

    def add_tensor(self, name: str, dims, ser):
        self.tensors.append((name, [int(d) for d in dims], int(ser[0]), bytes(ser[1])))
        return self

    @staticmethod
    def _meta_value(kind, v) -> bytes:
        if kind == "u32": return struct.pack("<II", UINT32, v)
        if kind == "i32": return struct.pack("<Ii", INT32, v)
        if kind == "u64": return struct.pack("<IQ", UINT64, v)
        if kind == "f32": return struct.pack("<If", FLOAT32, v)
        if kind == "bool": return struct.pack("<IB", BOOL, 1 if v else 0)
        if kind == "string": return struct.pack("<I", STRING) + _gguf_string(v)
        if kind == "arr_str": return struct.pack("<IIQ", ARRAY, STRING, len(v)) + b"".join(_gguf_string(s) for s in v)
        if kind == "arr_i32": return struct.pack("<IIQ", ARRAY, INT32, len(v)) + struct.pack(f"<{len(v)}i", *v)
        if kind == "arr_f32": return struct.pack("<IIQ", ARRAY, FLOAT32, len(v)) + struct.pack(f"<{len(v)}f", *v)
        raise ValueError(f"unknown metadata kind {kind}")

    def build(self) -> bytes:
        if not any(k == "general.alignment" for k, _, _ in self.meta):
            self.meta.append(("general.alignment", "u32", self.alignment))     # readers must agree with the padding
        al = self.alignment
        out = bytearray(struct.pack("<IIQQ", MAGIC, VERSION, len(self.tensors), len(self.meta)))
        for key, kind, v in self.meta:
            out += _gguf_string(key) + self._meta_value(kind, v)
        offsets, running = [], 0
        for _, _, _, data in self.tensors:          # offsets are relative to the data section, each aligned
            offsets.append(running)
            running += (len(data) + al - 1) // al * al
        for (name, dims, ttype, _), off in zip(self.tensors, offsets):
            out += _gguf_string(name) + struct.pack("<I", len(dims)) + struct.pack(f"<{len(dims)}Q", *dims)
            out += struct.pack("<IQ", ttype, off)
        out += b"\0" * (-len(out) % al)
        start = len(out)
        for (_, _, _, data), off in zip(self.tensors, offsets):
            out += b"\0" * (start + off - len(out))
            out += data
        out += b"\0" * (-len(out) % al)
        return bytes(out)


class GGUFFile:
    def __init__(self, version, alignment, metadata, tensors):
        self.version, self.alignment, self.metadata, self.tensors = version, alignment, metadata, tensors


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = memoryview(buf), 0

    def take(self, fmt):
        v = struct.unpack_from("<" + fmt, self.buf, self.pos)
        self.pos += struct.calcsize("<" + fmt)
        return v[0]

    def string(self):
        n = self.take("Q")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8")
        self.pos += n
        return s


def _read_meta_value(r: _Reader):
    t = r.take("I")
    # the 16-bit types are read four bytes wide, as the reference does (it never writes them)
    simple = {UINT8: "B", INT8: "b", UINT16: "I", INT16: "i", UINT32: "I", INT32: "i", FLOAT32: "f", UINT64: "Q",
              INT64: "q", FLOAT64: "d"}
    if t in simple:
        return r.take(simple[t])
    if t == BOOL:
        return r.take("B") != 0
    if t == STRING:
        return r.string()
    if t == ARRAY:
        et, n = r.take("I"), r.take("Q")
        if et == STRING:
            return [r.string() for _ in range(n)]
        if et in (INT32, UINT32, FLOAT32):
            return [r.take({INT32: "i", UINT32: "I", FLOAT32: "f"}[et]) for _ in range(n)]
        raise ValueError(f"Unsupported array elem type {et}")
    raise ValueError(f"Unsupported metadata type {t}")


def read_gguf(buf: bytes) -> GGUFFile:
    """Metadata (in file order), tensor infos and each tensor's raw bytes (up to the next tensor's offset, so the
    alignment padding comes along)."""
    r = _Reader(buf)
    if r.take("I") != MAGIC:
        raise ValueError("Not a GGUF file (bad magic)")
    version, n_tensors, n_meta = r.take("I"), r.take("Q"), r.take("Q")
    metadata = {}
    for _ in range(n_meta):
        key = r.string()
        metadata[key] = _read_meta_value(r)
    alignment = metadata.get("general.alignment", DEFAULT_ALIGNMENT)
    infos = []
    for _ in range(n_tensors):
        name = r.string()
        dims = [r.take("Q") for _ in range(r.take("I"))]
        infos.append(dict(name=name, dims=dims, type=r.take("I"), offset=r.take("Q")))
    start = r.pos + (-r.pos % alignment)
    for i, info in enumerate(infos):
        end = start + infos[i + 1]["offset"] if i + 1 < len(infos) else len(buf)
        info["data"] = bytes(r.buf[start + info["offset"]:end])
    return GGUFFile(version, alignment, metadata, infos)


# ---- what every architecture shares (arch/common.ts) ------------------------------------------------
_FILE_TYPE = {"f32": 0, "f16": 1, "q4_0": 2, "q8_0": 7}        # LLAMA_FTYPE, reported in general.file_type


def _token_types(tok: dict) -> list:
    special = set(tok.get("specials") or [])
    return [3 if (t.startswith("<|") and t.endswith("|>")) else 4 if t in special else 1 for t in tok["tokens"]]


def start_gguf(arch: str, tok: dict, quant: str, name=None, chat_template=None) -> GGUFWriter:
    """The general.* block and the tokenizer (byte-level BPE: model "gpt2", pre-tokenizer "qwen2"). `tok` is the
    reference's TokenizerData: tokens, merges, bosId, eosId, optional specials."""
    w = GGUFWriter()
    w.meta_string("general.architecture", arch)
    w.meta_string("general.name", name or f"gguf-trainer-{arch}")
    w.meta_u32("general.file_type", _FILE_TYPE[quant])
    w.meta_string("tokenizer.ggml.model", "gpt2")
    w.meta_string("tokenizer.ggml.pre", "qwen2")
    w.meta_arr_str("tokenizer.ggml.tokens", tok["tokens"])
    w.meta_arr_i32("tokenizer.ggml.token_type", _token_types(tok))
    w.meta_arr_str("tokenizer.ggml.merges", tok["merges"])
    w.meta_u32("tokenizer.ggml.bos_token_id", tok["bosId"])
    w.meta_u32("tokenizer.ggml.eos_token_id", tok["eosId"])
    w.meta_bool("tokenizer.ggml.add_bos_token", False)
    w.meta_bool("tokenizer.ggml.add_eos_token", False)
    if chat_template:
        w.meta_string("tokenizer.chat_template", chat_template)
    return w


def tokenizer_from_gguf(g: GGUFFile) -> dict:
    """load-gguf.ts:23-50: the token list, merges and the atomic specials (CONTROL and USER_DEFINED types, or the
    "<|...|>" shape when the file has no token_type)."""
    tokens, merges = g.metadata.get("tokenizer.ggml.tokens"), g.metadata.get("tokenizer.ggml.merges")
    if not isinstance(tokens, list) or not isinstance(merges, list):
        raise ValueError("GGUF missing tokenizer.ggml.tokens/merges")
    types = g.metadata.get("tokenizer.ggml.token_type")
    specials = [t for t, ty in zip(tokens, types) if ty in (3, 4)] if isinstance(types, list) else []
    if not specials:
        specials = [t for t in tokens if t.startswith("<|") and t.endswith("|>")]
    return dict(tokens=tokens, merges=merges, bosId=meta_num(g, "tokenizer.ggml.bos_token_id"),
                eosId=meta_num(g, "tokenizer.ggml.eos_token_id"), specials=specials or None)


def add_matrix(w: GGUFWriter, name: str, data: np.ndarray, quant: str):
    """[out, in] row-major here, so ggml's ne is [in, out]; block formats run along `in` and fall back to f16 when it
    is not a multiple of 32."""
    if data.ndim != 2:
        raise ValueError(f"addMatrix: {name} must be 2-D, got [{', '.join(map(str, data.shape))}]")
    out_dim, in_dim = data.shape
    q = "f16" if quant in ("q8_0", "q4_0") and in_dim % 32 != 0 else quant
    w.add_tensor(name, [in_dim, out_dim], serialize(data, q))


def add_vector(w: GGUFWriter, name: str, data: np.ndarray):
    if data.ndim != 1:
        raise ValueError(f"addVector: {name} must be 1-D, got [{', '.join(map(str, data.shape))}]")
    w.add_tensor(name, [data.shape[0]], serialize(data, "f32"))


def meta_num(g: GGUFFile, key: str):
    v = g.metadata.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ValueError(f'GGUF missing numeric metadata "{key}"')
    return v


def meta_num_or(g: GGUFFile, key: str, fallback):
    v = g.metadata.get(key)
    return v if isinstance(v, (int, float)) and not isinstance(v, bool) else fallback


def tensor_loader(g: GGUFFile):
    """load(name, shape) -> float32 array of that shape, dequantized per the tensor's own stored type; the file's
    dims (ggml order, trailing ones ignored) must be the shape reversed."""
    by_name = {t["name"]: t for t in g.tensors}

    def trim(d):
        d = list(d)
        while len(d) > 1 and d[-1] == 1:
            d.pop()
        return d

    def load(name: str, shape) -> np.ndarray:
        t = by_name.get(name)
        if t is None:
            raise ValueError(f'GGUF missing tensor "{name}"')
        want, have = trim(list(shape)[::-1]), trim(t["dims"])
        if want != have:
            raise ValueError(f'GGUF tensor "{name}" has dims [{", ".join(map(str, t["dims"]))}], but this model wants '
                             f'[{", ".join(map(str, want))}] (shape [{", ".join(map(str, shape))}] in this repo\'s order).')
        return dequantize(t["type"], t["data"], int(np.prod(shape))).reshape(shape)

    return load


def reorder_qk(w: np.ndarray, heads: int, head_dim: int, to_gguf: bool) -> np.ndarray:
    """llama only (llama.ts:104-129): this code rotates dimension j with j + head_dim/2, llama.cpp's llama graph
    rotates 2j with 2j+1, so inside every head row j goes to 2j and row j + half to 2j+1 on export, and back on
    load. Not idempotent: apply exactly once per direction."""
    half = head_dim // 2
    if heads * head_dim != w.shape[0] or head_dim % 2 != 0:
        raise ValueError(f"reorderQK: {heads} heads x {head_dim} dims does not tile {w.shape[0]} rows evenly")
    x = w.reshape(heads, head_dim, w.shape[1])
    out = np.empty_like(x)
    if to_gguf:
        out[:, 0::2], out[:, 1::2] = x[:, :half], x[:, half:]
    else:
        out[:, :half], out[:, half:] = x[:, 0::2], x[:, 1::2]
    return out.reshape(w.shape)


# ---- per-architecture names and keys ----------------------------------------------------------------
_TENSOR_NAME = {"attnNorm": "attn_norm", "qProj": "attn_q", "kProj": "attn_k", "vProj": "attn_v", "oProj": "attn_output",
                "qNorm": "attn_q_norm", "kNorm": "attn_k_norm", "postAttnNorm": "post_attention_norm",
                "ffnNorm": "ffn_norm", "gate": "ffn_gate", "up": "ffn_up", "down": "ffn_down",
                "postFfnNorm": "post_ffw_norm"}
# the order each exporter writes a layer's tensors in (llama.ts:396-409, qwen3.ts:381-394, gemma3.ts:448-463)
_EXPORT_ORDER = {
    "llama": ["attnNorm", "qProj", "kProj", "vProj", "oProj", "ffnNorm", "gate", "up", "down"],
    "qwen3": ["attnNorm", "qProj", "kProj", "vProj", "oProj", "qNorm", "kNorm", "ffnNorm", "gate", "up", "down"],
    "gemma3": ["attnNorm", "qProj", "kProj", "vProj", "qNorm", "kNorm", "oProj", "postAttnNorm", "ffnNorm", "gate", "up",
               "down", "postFfnNorm"],
}


def export_gguf(model: Model, tok: dict, quant: str = "f32", max_seq: int = 8192, name=None, chat_template=None) -> bytes:
    """The architecture's exportGGUF: metadata keys in the reference's order, then the tensors in its order.
    Matrices take `quant`, 1-D tensors stay f32."""
    if quant not in QUANT_NAMES:
        raise ValueError(f'unknown quant "{quant}" (valid: {", ".join(QUANT_NAMES)})')
    c, a = model.cfg, model.cfg.arch
    assert sorted(_EXPORT_ORDER[a]) == sorted(LAYER_KEYS[a])
    w = start_gguf(a, tok, quant, name, chat_template)
    w.meta_u32(f"{a}.context_length", max_seq)
    w.meta_u32(f"{a}.embedding_length", c.hidden)
    w.meta_u32(f"{a}.block_count", c.layers)
    w.meta_u32(f"{a}.feed_forward_length", c.ffn)
    w.meta_u32(f"{a}.attention.head_count", c.heads)
    w.meta_u32(f"{a}.attention.head_count_kv", c.kv_heads)
    w.meta_u32(f"{a}.attention.key_length", c.head_dim)
    w.meta_u32(f"{a}.attention.value_length", c.head_dim)
    w.meta_f32(f"{a}.attention.layer_norm_rms_epsilon", c.rms_eps)
    if a == "gemma3":
        w.meta_u32(f"{a}.attention.sliding_window", c.sliding_window)
        w.meta_u32(f"{a}.attention.sliding_window_pattern", c.swa_pattern)
        w.meta_f32(f"{a}.rope.freq_base", c.rope_base)
        w.meta_f32(f"{a}.rope.freq_base_swa", c.rope_base_local)
    else:
        w.meta_u32(f"{a}.rope.dimension_count", c.head_dim)
        w.meta_f32(f"{a}.rope.freq_base", c.rope_base)
    w.meta_u32(f"{a}.vocab_size", c.vocab)

    add_matrix(w, "token_embd.weight", model.tokenEmbd.data.reshape(model.tokenEmbd.shape), quant)
    add_vector(w, "output_norm.weight", model.outputNorm.data.reshape(-1))
    if model.output is not None:
        add_matrix(w, "output.weight", model.output.data.reshape(model.output.shape), quant)
    for i, L in enumerate(model.layers):
        for key in _EXPORT_ORDER[a]:
            t = L[key]
            data = t.data.reshape(t.shape)
            nm = f"blk.{i}.{_TENSOR_NAME[key]}.weight"
            if len(t.shape) == 1:
                add_vector(w, nm, data)
                continue
            if a == "llama" and key in ("qProj", "kProj"):
                data = reorder_qk(data, c.heads if key == "qProj" else c.kv_heads, c.head_dim, True)
            add_matrix(w, nm, data, quant)
    return w.build()


def config_from_gguf(g: GGUFFile):
    """(ModelConfig, max_seq) from the file's metadata, with each architecture's optional keys and fallbacks."""
    a = g.metadata.get("general.architecture")
    if a not in LAYER_KEYS:
        raise ValueError(f'GGUF general.architecture is "{a}"; this reader knows {", ".join(sorted(LAYER_KEYS))}')
    hidden, heads = meta_num(g, f"{a}.embedding_length"), meta_num(g, f"{a}.attention.head_count")
    tie = not any(t["name"] == "output.weight" for t in g.tensors)
    common = dict(arch=a, hidden=hidden, layers=meta_num(g, f"{a}.block_count"), heads=heads,
                  kv_heads=meta_num(g, f"{a}.attention.head_count_kv"), ffn=meta_num(g, f"{a}.feed_forward_length"),
                  rms_eps=meta_num(g, f"{a}.attention.layer_norm_rms_epsilon"), tie=tie)
    if a == "gemma3":
        cfg = ModelConfig(vocab=meta_num(g, f"{a}.vocab_size"), head_dim=meta_num(g, f"{a}.attention.key_length"),
                          rope_base=meta_num(g, f"{a}.rope.freq_base"), rope_base_local=meta_num(g, f"{a}.rope.freq_base_swa"),
                          sliding_window=meta_num(g, f"{a}.attention.sliding_window"),
                          swa_pattern=meta_num(g, f"{a}.attention.sliding_window_pattern"), **common)
    else:
        tokens = g.metadata.get("tokenizer.ggml.tokens")
        cfg = ModelConfig(vocab=meta_num_or(g, f"{a}.vocab_size", len(tokens) if isinstance(tokens, list) else 0),
                          head_dim=meta_num_or(g, f"{a}.attention.key_length", hidden // heads),
                          rope_base=meta_num_or(g, f"{a}.rope.freq_base", 10_000 if a == "llama" else 1_000_000), **common)
    return cfg, meta_num(g, f"{a}.context_length")


def load_weights(g: GGUFFile, cfg: ModelConfig) -> dict:
    """name -> float32 array for every parameter of the architecture (arch.param_names), llama's Q/K rows put back
    into this code's order."""
    load = tensor_loader(g)
    out = {"tokenEmbd": load("token_embd.weight", param_shape(cfg, "tokenEmbd")),
           "outputNorm": load("output_norm.weight", param_shape(cfg, "outputNorm"))}
    if not cfg.tie:
        out["output"] = load("output.weight", param_shape(cfg, "output"))
    for n in param_names(cfg):
        if "." not in n:
            continue
        layer, key = n.split(".", 1)
        wgt = load(f"blk.{layer[1:]}.{_TENSOR_NAME[key]}.weight", param_shape(cfg, n))
        if cfg.arch == "llama" and key in ("qProj", "kProj"):
            wgt = reorder_qk(wgt, cfg.heads if key == "qProj" else cfg.kv_heads, cfg.head_dim, False)
        out[n] = wgt
    return out


def load_model_from_gguf(buf: bytes):
    """load-gguf.ts:57-69: bytes -> (model with the file's weights, config, context length, tokenizer data)."""
    g = read_gguf(buf)
    cfg, max_seq = config_from_gguf(g)
    return Model(cfg, load_weights(g, cfg)), cfg, max_seq, tokenizer_from_gguf(g)


_MATCH_FIELDS = {
    "llama": [("vocab", "vocab"), ("hidden", "hidden"), ("layers", "layers"), ("heads", "heads"), ("kv_heads", "kv-heads"),
              ("head_dim", "head-dim"), ("ffn", "ffn-dim"), ("max_seq", "max-seq"), ("rms_eps", "rms-eps"),
              ("rope_base", "rope-base"), ("tie", "untied-embeddings")],
}
_MATCH_FIELDS["qwen3"] = _MATCH_FIELDS["llama"]


def config_matches(built: ModelConfig, ckpt: ModelConfig, built_max_seq=None, ckpt_max_seq=None, fields=None):
    """None when a run built with `built` can resume `ckpt`, else "<flag>: built X vs checkpoint Y" for the first
    difference (common.ts:196-214). Floats compare as the f32 the file can hold."""
    a = built.arch
    if fields is None:
        fields = _MATCH_FIELDS.get(a)
        if fields is None:      # gemma3.ts:491-512: head-dim is reported before the head count derived from it
            fields = [("vocab", "vocab"), ("hidden", "hidden"), ("layers", "layers"), ("head_dim", "head-dim"),
                      ("heads", "heads"), ("kv_heads", "kv-heads"), ("ffn", "ffn-dim"), ("max_seq", "max-seq"),
                      ("sliding_window", "window"), ("swa_pattern", "swa-pattern"), ("rms_eps", "rms-eps"),
                      ("rope_base", "rope-base"), ("rope_base_local", "rope-base-local"), ("tie", "untied-embeddings")]
    for key, flag in fields:
        if key == "max_seq":
            x, y = built_max_seq, ckpt_max_seq
            if x is None or y is None:
                continue
        else:
            x, y = getattr(built, key), getattr(ckpt, key)
        same = x == y or (isinstance(x, (int, float)) and isinstance(y, (int, float)) and not isinstance(x, bool)
                          and np.float32(x) == np.float32(y))
        if not same:
            show = (lambda v: str(not v).lower()) if key == "tie" else (lambda v: str(v))
            return f"{flag}: built {show(x)} vs checkpoint {show(y)}"
    return None
