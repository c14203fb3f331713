"""The checkpoint container of the w4g64 path (vpipe_amd/host/vpq_weights.h) against an
independent implementation of the format: the `safetensors` Python package reads what PackWriter
writes and PackFile reads what the package writes.  No GPU: these are host functions, driven
through the C test driver.  The layout rules checked are the reference's
(generative-models/quantize/safetensors-writer.cc: 16-byte aligned data section, odd-sized tensors
last, shards by a byte budget, model.safetensors.index.json)."""
import ctypes
import json
import os
import struct

import numpy as np
import pytest
import safetensors.numpy as stnp

import vpipe_amd

HERE = os.path.dirname(os.path.abspath(__file__))
NP_OF = {"U32": np.uint32, "F16": np.float16, "F32": np.float32, "U8": np.uint8, "I64": np.int64, "BF16": np.uint16}


@pytest.fixture(scope="module")
def drv():
    vpipe_amd.load()
    ctypes.CDLL(os.path.join(os.path.dirname(HERE), "vpipe_amd", "libvpq_host.so"), mode=ctypes.RTLD_GLOBAL)
    L = ctypes.CDLL(os.path.join(HERE, "host", "libhost_driver.so"))
    L.hw_open.restype = ctypes.c_void_p
    L.hw_open.argtypes = [ctypes.c_char_p, ctypes.c_ulonglong]
    L.hw_add.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_longlong), ctypes.c_int,
                         ctypes.c_void_p, ctypes.c_ulonglong]
    L.hw_close.argtypes = [ctypes.c_void_p]
    L.hr_open.restype = ctypes.c_void_p
    L.hr_open.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L.hr_why.restype = ctypes.c_char_p
    L.hr_close.argtypes = [ctypes.c_void_p]
    L.hr_count.argtypes = [ctypes.c_void_p]
    L.hr_name.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int]
    L.hr_info.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_longlong),
                          ctypes.POINTER(ctypes.c_ulonglong)]
    L.hr_read.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_ulonglong]
    L.hr_alignment.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_longlong)]
    L.hr_bits.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]
    L.hr_group.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]
    return L


def write_pack(drv, out_dir, tensors, shard_max=5 << 30):
    """tensors: list of (name, dtype string, numpy array)."""
    h = drv.hw_open(str(out_dir).encode(), shard_max)
    for name, dt, arr in tensors:
        arr = np.ascontiguousarray(arr)
        shape = (ctypes.c_longlong * arr.ndim)(*arr.shape)
        assert drv.hw_add(h, name.encode(), dt.encode(), shape, arr.ndim, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes) == 1
    assert drv.hw_close(h) == 1


class Reader:
    def __init__(self, drv, path, model_dir=False):
        self.L = drv
        self.h = drv.hr_open(str(path).encode(), 1 if model_dir else 0)
        self.why = drv.hr_why().decode(errors="replace")

    def ok(self):
        return bool(self.h)

    def names(self):
        out = []
        for i in range(self.L.hr_count(self.h)):
            buf = ctypes.create_string_buffer(512)
            assert self.L.hr_name(self.h, i, buf, 512) == 1
            out.append(buf.value.decode(errors="surrogateescape"))
        return out

    def info(self, name):
        dt = ctypes.create_string_buffer(16)
        shape = (ctypes.c_longlong * 8)()
        out = (ctypes.c_ulonglong * 4)()
        if self.L.hr_info(self.h, name.encode(errors="surrogateescape"), dt, shape, out) != 1:
            return None
        return {"dtype": dt.value.decode(errors="replace"), "shape": tuple(shape[i] for i in range(out[0])), "nbytes": out[1],
                "offset": out[2], "shard": out[3]}

    def read(self, name):
        i = self.info(name)
        buf = np.empty(i["nbytes"], dtype=np.uint8)
        assert self.L.hr_read(self.h, name.encode(), buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) == 1
        return buf.view(NP_OF[i["dtype"]]).reshape(i["shape"])

    def alignment(self):
        a = (ctypes.c_longlong * 4)()
        self.L.hr_alignment(self.h, a)
        return tuple(a)

    def close(self):
        if self.h:
            self.L.hr_close(self.h)
            self.h = None


def linear_tensors(rng, prefix, N, K):
    return [(prefix + ".weight", "U32", rng.integers(0, 2 ** 32, size=(N, K // 8), dtype=np.uint32)),
            (prefix + ".scales", "F16", rng.uniform(0.005, 0.02, size=(N, K // 64)).astype(np.float16)),
            (prefix + ".biases", "F16", rng.uniform(-0.2, -0.04, size=(N, K // 64)).astype(np.float16))]


def header_of(path):
    raw = open(path, "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    return n, json.loads(raw[8:8 + n]), len(raw)


def test_the_format_library_reads_what_the_writer_wrote(drv, tmp_path):
    rng = np.random.default_rng(1)
    tensors = linear_tensors(rng, "model.layers.0.mlp.down_proj", 48, 256)
    tensors.insert(1, ("model.layers.0.layer_scalar", "F16", np.array([1.5], dtype=np.float16)))   # 2 bytes: odd-sized
    tensors.append(("model.norm.weight", "F32", rng.normal(size=(40,)).astype(np.float32)))
    tensors.append(('odd "name"\\x', "U8", np.arange(7, dtype=np.uint8)))
    write_pack(drv, tmp_path, tensors)
    files = sorted(f for f in os.listdir(tmp_path) if f.endswith(".safetensors"))
    assert files == ["model-00001-of-00001.safetensors"]
    assert not [f for f in os.listdir(tmp_path) if f.endswith(".tmp")]
    path = tmp_path / files[0]
    got = stnp.load_file(str(path))
    assert sorted(got) == sorted(n for n, _, _ in tensors)
    for name, dt, arr in tensors:
        assert got[name].dtype == arr.dtype and got[name].shape == arr.shape
        assert np.array_equal(got[name], arr)
    hlen, hdr, _ = header_of(path)
    assert (8 + hlen) % 16 == 0                                   # data section on a 16-byte boundary
    # tensors whose size is a multiple of 16 sit on 16-byte offsets; the odd ones come last
    offs = {n: hdr[n]["data_offsets"] for n in hdr}
    for name, _, arr in tensors:
        if arr.nbytes % 16 == 0:
            assert offs[name][0] % 16 == 0, name
    last_even = max(offs[n][1] for n, _, a in tensors if a.nbytes % 16 == 0)
    assert all(offs[n][0] >= last_even for n, _, a in tensors if a.nbytes % 16 != 0)
    # the byte ranges tile the blob without gaps
    spans = sorted(offs.values())
    assert spans[0][0] == 0 and all(spans[i][1] == spans[i + 1][0] for i in range(len(spans) - 1))
    index = json.load(open(tmp_path / "model.safetensors.index.json"))
    assert index["weight_map"] == {n: files[0] for n, _, _ in tensors}
    assert index["metadata"]["total_size"] == sum(a.nbytes for _, _, a in tensors)


def test_writer_shards_by_budget_and_the_reader_merges_them(drv, tmp_path):
    rng = np.random.default_rng(2)
    tensors = []
    for layer in range(5):
        tensors += linear_tensors(rng, "model.layers.%d.self_attn.q_proj" % layer, 64, 512)     # 16 KB + 1 KB + 1 KB
    write_pack(drv, tmp_path, tensors, shard_max=40 << 10)
    files = sorted(f for f in os.listdir(tmp_path) if f.endswith(".safetensors"))
    assert len(files) == 3 and files[0] == "model-00001-of-00003.safetensors"
    index = json.load(open(tmp_path / "model.safetensors.index.json"))
    r = Reader(drv, tmp_path, model_dir=True)
    assert r.ok(), r.why
    assert r.names() == sorted(n for n, _, _ in tensors)
    for name, dt, arr in tensors:
        i = r.info(name)
        assert i["dtype"] == dt and i["shape"] == arr.shape and i["nbytes"] == arr.nbytes
        assert files[i["shard"]] == index["weight_map"][name]
        assert np.array_equal(r.read(name), arr)
    assert r.alignment() == (15, 0, 3, 0)
    assert drv.hr_bits(r.h, b"model.layers.3.self_attn.q_proj", 512) == 4
    assert drv.hr_group(r.h, b"model.layers.3.self_attn.q_proj", 512) == 64
    assert drv.hr_bits(r.h, b"model.layers.9.self_attn.q_proj", 512) == 0
    r.close()
    # a duplicate name and an add after close are refused
    h = drv.hw_open(str(tmp_path / "dup").encode(), 1 << 30)
    a = np.zeros(4, dtype=np.float32)
    shape = (ctypes.c_longlong * 1)(4)
    assert drv.hw_add(h, b"t", b"F32", shape, 1, a.ctypes.data_as(ctypes.c_void_p), 16) == 1
    assert drv.hw_add(h, b"t", b"F32", shape, 1, a.ctypes.data_as(ctypes.c_void_p), 16) == 0
    assert drv.hw_close(h) == 1


def test_the_reader_reads_what_the_format_library_wrote(drv, tmp_path):
    rng = np.random.default_rng(3)
    tensors = {n: a for n, _, a in linear_tensors(rng, "lm_head", 80, 192)}
    tensors["w8.weight"] = rng.integers(0, 2 ** 32, size=(16, 64), dtype=np.uint32)       # 8-bit, K = 256
    tensors["w8.scales"] = np.ones((16, 8), dtype=np.float16)                             # group 32
    tensors["w8.biases"] = np.zeros((16, 8), dtype=np.float16)
    tensors["step"] = np.array(7, dtype=np.int64)                                         # rank 0
    path = tmp_path / "model.safetensors"
    stnp.save_file(tensors, str(path), metadata={"format": "pt", "note": 'quote " and \\ backslash'})
    for opener in ((path, False), (tmp_path, True)):
        r = Reader(drv, *opener)
        assert r.ok(), r.why
        assert r.names() == sorted(tensors)                       # __metadata__ is not a tensor
        for name, arr in tensors.items():
            got = r.read(name)
            assert got.dtype == arr.dtype and got.shape == arr.shape and np.array_equal(got, arr)
        hlen, _, _ = header_of(path)
        t, mis, shards, bad = r.alignment()
        assert (t, shards) == (len(tensors), 1) and bad == (0 if (8 + hlen) % 16 == 0 else 1)
        assert (drv.hr_bits(r.h, b"lm_head", 192), drv.hr_group(r.h, b"lm_head", 192)) == (4, 64)
        assert (drv.hr_bits(r.h, b"w8", 256), drv.hr_group(r.h, b"w8", 256)) == (8, 32)
        r.close()


def test_malformed_files_are_refused(drv, tmp_path):
    good = tmp_path / "good.safetensors"
    stnp.save_file({"a": np.arange(8, dtype=np.float32)}, str(good))
    raw = open(good, "rb").read()
    hlen = struct.unpack("<Q", raw[:8])[0]

    def attempt(name, data):
        p = tmp_path / name
        open(p, "wb").write(data)
        r = Reader(drv, p)
        ok, why = r.ok(), r.why
        r.close()
        return ok, why

    assert attempt("same.safetensors", raw)[0]
    assert not attempt("short.safetensors", raw[:5])[0]
    assert not attempt("hlen.safetensors", struct.pack("<Q", len(raw)) + raw[8:])[0]          # header past the end
    assert not attempt("trunc.safetensors", raw[:-4])[0]                                      # data range past the end
    assert not attempt("notjson.safetensors", raw[:8] + b"[" + raw[9:])[0]
    hdr = json.loads(raw[8:8 + hlen])
    hdr["a"]["shape"] = [9]                                                                   # disagrees with the bytes
    h2 = json.dumps(hdr).encode()
    ok, why = attempt("shape.safetensors", struct.pack("<Q", len(h2)) + h2 + raw[8 + hlen:])
    assert not ok and "dtype and shape" in why
    assert not Reader(drv, tmp_path / "absent.safetensors").ok()
    assert not Reader(drv, tmp_path / "no_such_dir", model_dir=True).ok()
    # an index that points outside the directory, or at a shard without the tensor
    d = tmp_path / "m"
    os.makedirs(d)
    stnp.save_file({"a": np.arange(8, dtype=np.float32)}, str(d / "s1.safetensors"))
    json.dump({"weight_map": {"a": "../good.safetensors"}}, open(d / "model.safetensors.index.json", "w"))
    assert not Reader(drv, d, model_dir=True).ok()
    json.dump({"weight_map": {"b": "s1.safetensors"}}, open(d / "model.safetensors.index.json", "w"))
    assert not Reader(drv, d, model_dir=True).ok()
    json.dump({"weight_map": {"a": "s1.safetensors"}}, open(d / "model.safetensors.index.json", "w"))
    r = Reader(drv, d, model_dir=True)
    assert r.ok(), r.why
    r.close()


def test_mutated_headers_never_crash_the_reader(drv, tmp_path):
    # whatever a damaged header says, the reader answers (tensors stay inside the file) or refuses
    src = tmp_path / "src.safetensors"
    stnp.save_file({"a.weight": np.arange(64, dtype=np.uint32).reshape(4, 16), "a.scales": np.ones((4, 2), np.float16),
                    "a.biases": np.ones((4, 2), np.float16)}, str(src), metadata={"k": "v"})
    raw = bytearray(open(src, "rb").read())
    hlen = struct.unpack("<Q", raw[:8])[0]
    rng = np.random.default_rng(11)
    p = tmp_path / "mut.safetensors"
    opened = 0
    for _ in range(300):
        m = bytearray(raw)
        for _ in range(int(rng.integers(1, 4))):
            pos = int(rng.integers(0, 8 + hlen))
            m[pos] = int(rng.integers(0, 256)) if rng.random() < 0.5 else ord(rng.choice(list('{}[]",:0189 \\')))
        open(p, "wb").write(m)
        r = Reader(drv, p)
        if r.ok():
            opened += 1
            for name in r.names():
                i = r.info(name)
                assert i is not None and i["offset"] + i["nbytes"] <= len(m)
                buf = np.empty(i["nbytes"], dtype=np.uint8)
                assert drv.hr_read(r.h, name.encode(errors="surrogateescape"), buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes) == 1
        r.close()
    assert 0 < opened < 300
