"""GGUF reader of the library (include/qk_gguf.h) on synthetic files: what the reference's reader
accepts (src/gguf.h:54-198: v2/v3, alignment, integer and string metadata, split shards) is read
back byte for byte; what it would read out of bounds is an error here.  Host code only."""
import os
import struct

import numpy as np
import pytest


@pytest.fixture(scope="module")
def small_layer(qk):
    return qk.synth.HostLayer(seed=11, n_embd=256, n_ff=256, n_expert=4, n_used=2)


KVS = {"general.architecture": "qwen3next", "qwen3next.expert_used_count": 2, "qwen3next.block_count": 48,
       "tokenizer.ggml.tokens": ["<a>", "b", ""], "tokenizer.ggml.token_type": [1, 2, 3], "some.float": 0.25,
       "some.bool": True, "some.big": 2 ** 40}


def as_bytes(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


@pytest.mark.parametrize("version,alignment", [(3, 32), (2, 32), (3, 64), (3, 4096)])
def test_round_trip(qk, small_layer, tmp_path, version, alignment):
    p = tmp_path / "m.gguf"
    tensors = qk.gguf.layer_tensors(small_layer, 7) + [("output_norm.weight", qk.F32, (256,), np.arange(256, dtype=np.float32)),
                                                       ("odd.type", 30, (8, 2), np.zeros(32, dtype=np.uint8))]
    qk.gguf.write(p, KVS, tensors, alignment=alignment, version=version)
    with qk.gguf.File(p) as f:
        assert (f.version, f.n_shards, len(f)) == (version, 1, len(tensors))
        assert f.names() == sorted(t[0] for t in tensors)
        assert f.kv_str("general.architecture") == "qwen3next"
        assert f.kv_int("qwen3next.expert_used_count") == 2 and f.kv_int("some.big") == 2 ** 40
        assert f.kv_int("some.bool") == 1
        assert f.kv_int("missing", default=5) == 5 and f.kv_str("missing", default="x") == "x"
        with pytest.raises(qk.QkError) as e:      # floats and arrays are skipped, as in the reference
            f.kv_int("some.float")
        assert e.value.code == qk.gguf.ENOTFOUND
        for name, type_, ne, data in tensors:
            t = f.find(name)
            assert (t.type, t.n_dims) == (type_, len(ne)) and t.ne[:len(ne)] == tuple(ne) and t.ne[len(ne):] == (1,) * (4 - len(ne))
            if type_ == 30:                       # a type whose row size the library does not know
                assert t.nbytes == 0
                continue
            assert np.array_equal(t.bytes(), as_bytes(data)), name
        with pytest.raises(qk.QkError) as e:
            f.find("nope")
        assert e.value.code == qk.gguf.ENOTFOUND
        dims, ts = f.moe_tensors(7)
        assert dims == dict(n_embd=256, n_ff=256, n_expert=4, n_used=2, gu_type=qk.IQ3_XXS, down_type=qk.IQ4_XS)
        assert np.array_equal(ts["down_exps"].bytes(), as_bytes(small_layer.down_exps))


def test_split_shards(qk, small_layer, tmp_path):
    ts = qk.gguf.layer_tensors(small_layer, 0)
    first, second = tmp_path / "m-00001-of-00002.gguf", tmp_path / "m-00002-of-00002.gguf"
    qk.gguf.write(first, dict(KVS, **{"split.count": 2, "split.tensors.count": 8}), ts[:3])
    qk.gguf.write(second, {"split.no": 1}, ts[3:], alignment=64)
    with qk.gguf.File(first) as f:
        assert f.n_shards == 2 and len(f) == 8
        assert f.find(ts[5][0]).shard == 1 and f.find(ts[0][0]).shard == 0
        for name, _, _, data in ts:
            assert np.array_equal(f.find(name).bytes(), as_bytes(data))
        assert f.kv_int("split.no", default=99) == 99          # metadata comes from the first shard only
    # a first shard under another name, a missing sibling, a wrong total
    other = tmp_path / "renamed.gguf"
    other.write_bytes(first.read_bytes())
    with pytest.raises(qk.QkError):
        qk.gguf.File(other)
    second.unlink()
    with pytest.raises(qk.QkError) as e:
        qk.gguf.File(first)
    assert e.value.code == qk.gguf.EIO
    qk.gguf.write(second, {}, ts[3:7])
    with pytest.raises(qk.QkError) as e:
        qk.gguf.File(first)
    assert e.value.code == qk.gguf.EFORMAT


def test_malformed_files_are_errors(qk, small_layer, tmp_path):
    good = tmp_path / "good.gguf"
    qk.gguf.write(good, KVS, qk.gguf.layer_tensors(small_layer, 1))
    raw = good.read_bytes()
    bad = tmp_path / "bad.gguf"

    def expect(data, code=None):
        bad.write_bytes(data)
        with pytest.raises(qk.QkError) as e:
            qk.gguf.File(bad)
        if code is not None:
            assert e.value.code == code, str(e.value)

    with pytest.raises(qk.QkError) as e:
        qk.gguf.File(tmp_path / "absent.gguf")
    assert e.value.code == qk.gguf.EIO
    expect(b"", qk.gguf.EFORMAT)
    expect(b"GGML" + raw[4:], qk.gguf.EFORMAT)
    expect(raw[:4] + struct.pack("<I", 1) + raw[8:], qk.gguf.EFORMAT)        # version 1
    expect(raw[:4] + struct.pack("<I", 4) + raw[8:], qk.gguf.EFORMAT)        # version 4
    expect(raw[:8] + struct.pack("<Q", 2 ** 60) + raw[16:], qk.gguf.EFORMAT)  # tensor count
    expect(raw[:16] + struct.pack("<Q", 2 ** 60) + raw[24:], qk.gguf.EFORMAT)  # key count
    # the header region cut anywhere: an error, never a read past the mapping
    header_len = raw.index(as_bytes(small_layer.down_exps)[:64].tobytes())     # somewhere past the directory
    for cut in list(range(24, 200, 7)) + list(range(200, header_len, 97)):
        expect(raw[:cut])
    # data section cut short: some tensor runs past the end
    expect(raw[:len(raw) - 1], qk.gguf.EFORMAT)
    expect(raw[:header_len + 10], qk.gguf.EFORMAT)


def test_corrupted_bytes_never_crash(qk, small_layer, tmp_path):
    """Seeded byte flips in the header region: the reader returns a file or an error."""
    good = tmp_path / "good.gguf"
    qk.gguf.write(good, KVS, qk.gguf.layer_tensors(small_layer, 1))
    raw = bytearray(good.read_bytes())
    header_len = bytes(raw).index(as_bytes(small_layer.down_exps)[:64].tobytes())
    rng = np.random.default_rng(2024)
    bad = tmp_path / "bad.gguf"
    opened = failed = 0
    for _ in range(300):
        b = bytearray(raw)
        for _ in range(int(rng.integers(1, 4))):
            b[int(rng.integers(4, header_len))] = int(rng.integers(0, 256))
        bad.write_bytes(bytes(b))
        try:
            with qk.gguf.File(bad) as f:
                for i in range(len(f)):
                    t = f.tensor_at(i)
                    if t.nbytes:
                        t.bytes()[-1]           # the last byte of every tensor is inside the mapping
                opened += 1
        except qk.QkError:
            failed += 1
    assert opened + failed == 300 and failed > 0


def test_alignment_must_be_a_power_of_two(qk, tmp_path):
    p = tmp_path / "a.gguf"
    qk.gguf.write(p, {"general.alignment": 48}, [("t", qk.F32, (4,), np.zeros(4, dtype=np.float32))])
    with pytest.raises(qk.QkError) as e:
        qk.gguf.File(p)
    assert e.value.code == qk.gguf.EFORMAT


def test_moe_layer_checks(qk, small_layer, tmp_path):
    """The reference's loader checks (src/main.cpp:1278-1301) and the shape checks added here."""
    base = qk.gguf.layer_tensors(small_layer, 2)
    p = tmp_path / "l.gguf"

    def load(tensors, kvs=KVS):
        qk.gguf.write(p, kvs, tensors)
        with qk.gguf.File(p) as f:
            return f.moe_tensors(2)[0]

    assert load(base)["n_used"] == 2
    with pytest.raises(qk.QkError) as e:                  # default top-8 with four experts
        load(base, {"general.architecture": "x"})
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:                  # missing tensor
        load(base[:-1])
    assert e.value.code == qk.gguf.ENOTFOUND
    wrong_type = [(n, (qk.Q6_K if "gate_exps" in n else t), ne, d) for n, t, ne, d in base]
    with pytest.raises(qk.QkError) as e:
        load(wrong_type)
    assert e.value.code == -3
    name, t, ne, d = base[4]                              # down_exps with the dimensions swapped
    wrong_shape = base[:4] + [(name, t, (ne[0], 2 * ne[1], ne[2] // 2), d)] + base[5:]   # same bytes, other shape
    with pytest.raises(qk.QkError) as e:
        load(wrong_shape)
    assert e.value.code == -2
    with pytest.raises(qk.QkError) as e:                  # top-k above the selector's 16
        load(base, dict(KVS, **{"qwen3next.expert_used_count": 17}))
    assert e.value.code == -2


def test_fused_ssm_ba_rows(qk, tmp_path):
    """The fused decay / write-strength tensor of qwen3next files (reference src/main.cpp:3936-3948):
    per key-head group g the rows 4g, 4g+1 are beta of the value heads 2g, 2g+1 and the rows 4g+2, 4g+3
    their alpha.  The synthetic writer interleaves by that rule, split_ba undoes it, and a whole-model
    file written with the fused form holds ssm_ba [n_embd, 64] in place of the two split tensors."""
    FM = qk.engine.FullModel
    hv = 32
    alpha = np.arange(hv, dtype=np.float32)[:, None] + np.zeros((1, 4), np.float32)          # row h holds h
    beta = 100 + np.arange(hv, dtype=np.float32)[:, None] + np.zeros((1, 4), np.float32)     # row h holds 100 + h
    ba = FM.interleave_ba(alpha, beta)
    assert ba[:8, 0].tolist() == [100, 101, 0, 1, 102, 103, 2, 3]
    assert ba[60:, 0].tolist() == [130, 131, 30, 31]
    a2, b2 = FM.split_ba(ba)
    assert np.array_equal(a2, alpha) and np.array_equal(b2, beta)
    for type_, nbytes in ((qk.F32, 64 * 2048 * 4), (qk.Q8_0, 64 * 2176)):
        model = FM(3, kinds="R", vocab=64, fused_ba=type_)
        path = model.write(str(tmp_path / f"fused_{type_}.gguf"))
        with qk.gguf.File(path) as f:
            names = f.names()
            assert "blk.0.ssm_alpha.weight" not in names and "blk.0.ssm_beta.weight" not in names
            t = f.find("blk.0.ssm_ba.weight")
            assert (t.type, tuple(t.ne[:2]), t.nbytes) == (type_, (2048, 64), nbytes)
