"""A reader for GGUF files, enough to feed real checkpoints to the kernels: header, metadata, tensor
table, and memory-mapped tensor bytes handed to ``frink_amd.Weights`` without a copy on the host.

Mirrors the reference's parser (crates/frink-gguf/src/lib.rs:429-560): versions 2 and 3, little
endian; a tensor's shape lists its innermost dimension first (``shape[0]`` = columns of a weight
matrix); tensor data starts at the next ``general.alignment`` boundary (default 32, must be a power
of two) behind the tensor table, and a tensor's ``offset`` counts from there.  The same refusals:
bad magic, unknown version, an alignment that is not a power of two, a tensor that declares more
elements than eight times the file's bytes, a tensor whose bytes run past the end of the file.
"""
import mmap
import struct

import numpy as np

GGUF_MAGIC = 0x46554747  # "GGUF"

# ggml type tag -> (name, block bytes, block elements) for the types whose byte size this reader knows
GGML_TYPES = {
    0: ("F32", 4, 1), 1: ("F16", 2, 1), 2: ("Q4_0", 18, 32), 3: ("Q4_1", 20, 32), 6: ("Q5_0", 22, 32),
    7: ("Q5_1", 24, 32), 8: ("Q8_0", 34, 32), 10: ("Q2_K", 84, 256), 11: ("Q3_K", 110, 256),
    12: ("Q4_K", 144, 256), 13: ("Q5_K", 176, 256), 14: ("Q6_K", 210, 256), 30: ("BF16", 2, 1),
}


class GgufError(ValueError):
    pass


class TensorInfo:
    def __init__(self, name, shape, type_tag, offset):
        self.name, self.shape, self.type_tag, self.offset = name, tuple(shape), type_tag, offset

    @property
    def type_name(self):
        return GGML_TYPES.get(self.type_tag, ("type %d" % self.type_tag,))[0]

    @property
    def n_elements(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    @property
    def byte_len(self):
        """Bytes of the tensor, or None for a type of unknown size or a row that is not whole blocks."""
        t = GGML_TYPES.get(self.type_tag)
        if t is None or not self.shape or self.shape[0] % t[2]:
            return None
        return self.n_elements // t[2] * t[1]

    def __repr__(self):
        return "TensorInfo(%r, %s, %s, offset=%d)" % (self.name, self.shape, self.type_name, self.offset)


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GgufError("the file ends inside its header (offset %d)" % self.pos)
        v = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v[0]

    def string(self):
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GgufError("a string of %d bytes runs past the end of the file" % n)
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", "replace")
        self.pos += n
        return s

    _SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}

    def value(self, tag=None):
        tag = self.take("<I") if tag is None else tag
        if tag in self._SCALARS:
            return self.take(self._SCALARS[tag])
        if tag == 8:
            return self.string()
        if tag == 9:
            elem, count = self.take("<I"), self.take("<Q")
            if count > len(self.buf):
                raise GgufError("an array of %d elements cannot fit the file" % count)
            return [self.value(elem) for _ in range(count)]
        raise GgufError("unknown metadata value type %d" % tag)


class GgufFile:
    """An open GGUF file: ``metadata`` (dict), ``tensors`` (list of TensorInfo), ``tensor_bytes(name)``."""

    def __init__(self, path):
        self._fh = open(path, "rb")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        buf = memoryview(self._map)
        c = _Cursor(buf)
        magic = c.take("<I")
        if magic != GGUF_MAGIC:
            raise GgufError("bad magic 0x%08x" % magic)
        self.version = c.take("<I")
        if self.version not in (2, 3):
            raise GgufError("unsupported GGUF version %d" % self.version)
        n_tensors, n_kv = c.take("<Q"), c.take("<Q")
        self.metadata = {}
        for _ in range(n_kv):
            key = c.string()
            self.metadata[key] = c.value()
        self.tensors = []
        for _ in range(n_tensors):
            name = c.string()
            n_dims = c.take("<I")
            shape = [c.take("<Q") for _ in range(n_dims)]
            info = TensorInfo(name, shape, c.take("<I"), c.take("<Q"))
            if info.n_elements > len(buf) * 8:
                raise GgufError("tensor %r declares shape %s, more than a file of %d bytes can hold"
                                % (name, info.shape, len(buf)))
            self.tensors.append(info)
        align = self.metadata.get("general.alignment", 32)
        if not isinstance(align, int) or align <= 0 or align & (align - 1):
            raise GgufError("general.alignment is %r: it must be a power of two" % (align,))
        self.data_start = (c.pos + align - 1) // align * align
        self._by_name = {t.name: t for t in self.tensors}

    def close(self):
        """Closes the file.  Arrays handed out by tensor_bytes keep the mapping alive: it then goes away
        with the last of them."""
        try:
            self._map.close()
        except BufferError:
            pass
        self._fh.close()

    def info(self, name):
        if name not in self._by_name:
            raise GgufError("no tensor named %r" % name)
        return self._by_name[name]

    def tensor_bytes(self, name):
        """The tensor's bytes as a read-only uint8 array over the mapped file (no copy)."""
        t = self.info(name)
        n = t.byte_len
        if n is None:
            raise GgufError("tensor %r has type %s, whose size is not known here" % (name, t.type_name))
        start = self.data_start + t.offset
        if start + n > len(self._map):
            raise GgufError("tensor %r needs %d bytes, the file has %d left" % (name, n, max(0, len(self._map) - start)))
        return np.frombuffer(self._map, dtype=np.uint8, count=n, offset=start)

    def weights(self, name):
        """The 2-D tensor `name` as resident device weights (rows = shape[1], cols = shape[0]); its kind
        must be one the library has kernels for."""
        import frink_amd as fa
        t = self.info(name)
        if len(t.shape) != 2:
            raise GgufError("tensor %r has shape %s, not a matrix" % (name, t.shape))
        if fa.matvec_kernel(t.type_tag) is None:
            raise GgufError("tensor %r is %s: no kernel for that kind" % (name, t.type_name))
        cols, rows = t.shape
        return fa.Weights.from_host(t.type_tag, self.tensor_bytes(name), rows, cols)


def write_gguf(path, metadata, tensors, alignment=32, version=3):
    """Writes a GGUF file (for tests and tools): `metadata` maps keys to int / float / bool / str values,
    `tensors` is a list of (name, shape innermost first, ggml type tag, bytes-like)."""
    def s(text):
        b = text.encode()
        return struct.pack("<Q", len(b)) + b

    def v(val):
        if isinstance(val, bool):
            return struct.pack("<I?", 7, val)
        if isinstance(val, int):
            return struct.pack("<II", 4, val) if 0 <= val < 1 << 32 else struct.pack("<Iq", 11, val)
        if isinstance(val, float):
            return struct.pack("<If", 6, val)
        return struct.pack("<I", 8) + s(str(val))

    meta = dict(metadata)
    meta.setdefault("general.alignment", alignment)
    head = struct.pack("<IIQQ", GGUF_MAGIC, version, len(tensors), len(meta))
    for k, val in meta.items():
        head += s(k) + v(val)
    offset, infos, blobs = 0, b"", []
    for name, shape, tag, data in tensors:
        data = bytes(data)
        infos += s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        infos += struct.pack("<IQ", tag, offset)
        pad = -len(data) % alignment
        blobs.append(data + bytes(pad))
        offset += len(data) + pad
    head += infos
    head += bytes(-len(head) % alignment)
    with open(path, "wb") as f:
        f.write(head)
        for b in blobs:
            f.write(b)
