"""Host-side rows either side of the operators: the ternarise+pack producer and the .tllm reader /
synthetic writer. Everything but the last test runs without a GPU (host functions of the C ABI).

The producer is checked against the known-answer words of the reference's own packing test
(tests/test_packing.py:55-81), its two degenerate cases (test_packing.py:177-205), closed forms, and
bit for bit against the oracle's restatement of ternarize/pack.py. The file layout is checked by
parsing the written file independently in numpy (header fields, array order and sizes of reference
src/model.cpp:72-212)."""
import os
import struct

import numpy as np
import pytest

import ternary_llm_amd as tl
from tests import synth


def test_pack_known_answer_words():
    # row 0 = {+1@0, -1@1, +1@31, -1@32, -1@63}; row 1 alternating +1/-1 (reference test_packing.py:55-81)
    w = np.zeros((2, 128), np.float32)
    w[0, [0, 31]] = 1.0
    w[0, [1, 32, 63]] = -1.0
    w[1, 0::2] = 1.0
    w[1, 1::2] = -1.0
    nz, sg, sc = tl.ternarize_pack(w)
    assert nz[0, 0] == 0x80000003 and sg[0, 0] == 0x80000001
    assert nz[0, 1] == 0x80000001 and sg[0, 1] == 0
    assert nz[0, 2] == 0 and nz[0, 3] == 0
    assert (nz[1] == 0xFFFFFFFF).all() and (sg[1] == 0x55555555).all()
    assert sc[0, 0] == np.float16(1.0) and sc[1, 0] == np.float16(1.0)


def test_ternarize_degenerate_and_closed_forms():
    nz, sg, sc = tl.ternarize_pack(np.zeros((3, 256), np.float32))
    assert not nz.any() and not sg.any() and (sc == 0).all()      # all-zero group: scale 0
    w = np.full((1, 128), 0.25, np.float32)
    w[0, ::3] *= -1
    nz, sg, sc = tl.ternarize_pack(w)                              # uniform magnitude: everything survives
    assert (nz == 0xFFFFFFFF).all() and sc[0, 0] == np.float16(0.25)
    assert np.array_equal(synth.unpack_np(nz, sg)[0], np.sign(w[0]).astype(np.int8))
    # threshold = 0.7 * mean|w|: with 127 entries of 1 and one of 0.5, mean = 0.99609, thr = 0.697 -> 0.5 dies
    w = np.ones((1, 128), np.float32)
    w[0, 77] = 0.5
    nz, sg, sc = tl.ternarize_pack(w)
    t = synth.unpack_np(nz, sg)[0]
    assert t[77] == 0 and t.sum() == 127 and sc[0, 0] == np.float16(1.0)
    # a threshold factor of 0 keeps every non-zero entry; scale = mean |w|
    w = np.random.default_rng(5).standard_normal((4, 256)).astype(np.float32)
    nz, sg, sc = tl.ternarize_pack(w, threshold_factor=0.0)
    assert np.array_equal(synth.unpack_np(nz, sg), np.sign(w).astype(np.int8))
    want = np.abs(w).reshape(4, 2, 128).astype(np.float64).mean(axis=2)
    assert np.allclose(sc.astype(np.float64), want, rtol=2e-3)


@pytest.mark.parametrize("rows,cols,group", [(5, 128, 128), (64, 1024, 128), (7, 256, 64), (3, 512, 256)])
def test_ternarize_pack_matches_oracle_bit_for_bit(oracle, rows, cols, group):
    w = (0.02 * np.random.default_rng(rows * cols).standard_normal((rows, cols))).astype(np.float32)
    nz, sg, sc = tl.ternarize_pack(w, group_size=group)
    t, s = oracle.ternarize(w, group=group)
    onz, osg = oracle.pack(t.reshape(rows, cols))
    assert np.array_equal(nz, onz) and np.array_equal(sg, osg)
    assert np.array_equal(sc.view(np.uint16).ravel(), np.asarray(s).view(np.uint16).ravel())


def _pack_fixture(name):
    import json
    with open(os.path.join(os.path.dirname(__file__), "golden", name + ".json")) as f:
        fx = json.load(f)
    rows, cols = fx["rows"], fx["cols"]
    w = np.array([int(v, 16) for v in fx["weight_f32"]], np.uint32).view(np.float32).reshape(rows, cols)
    t = np.array(["-0+".index(c) - 1 for c in fx["ternary"]], np.int8).reshape(rows, cols)
    nz = np.array([int(v, 16) for v in fx["nz"]], np.uint32).reshape(rows, cols // 32)
    sg = np.array([int(v, 16) for v in fx["sign"]], np.uint32).reshape(rows, cols // 32)
    sc = np.array([int(v, 16) for v in fx["scales"]], np.uint16).reshape(rows, cols // fx["group"])
    return fx, w, t, nz, sg, sc


@pytest.mark.parametrize("name", ["pack_seed42", "pack_seed123"])
def test_producer_reproduces_the_reference_producer(oracle, name):
    """tests/golden/pack_seed*.json hold what the reference's ternarize_tensor + pack_ternary_to_bitmasks
    (ternarize/pack.py:41-101, 120-169) gave for the two seeded tensors of its own packing test
    (tests/test_packing.py:92-111, 141-173), written by tests/golden/make_pack_fixtures.py. The C++ producer
    and the oracle's restatement must give the same masks AND the same fp16 scales, bit for bit (the
    reference sums a group in torch's order, both restatements left to right: on these 320 groups the
    fp32 sums round to the same fp16 value)."""
    fx, w, t, rnz, rsg, rsc = _pack_fixture(name)
    nz, sg, sc = tl.ternarize_pack(w, group_size=fx["group"], threshold_factor=fx["threshold_factor"])
    assert np.array_equal(nz, rnz) and np.array_equal(sg, rsg)
    assert np.array_equal(sc.view(np.uint16), rsc)
    ot, os_ = oracle.ternarize(w, group=fx["group"], factor=fx["threshold_factor"])
    assert np.array_equal(ot.reshape(t.shape), t)
    assert np.array_equal(np.asarray(os_).view(np.uint16).reshape(rsc.shape), rsc)
    onz, osg = oracle.pack(t)
    assert np.array_equal(onz, rnz) and np.array_equal(osg, rsg)
    assert np.array_equal(synth.unpack_np(rnz, rsg), t)      # the independent unpack of tests/synth.py


def test_ternarize_rejects_bad_shapes():
    with pytest.raises(tl.TllmError):
        tl.ternarize_pack(np.zeros((2, 100), np.float32))          # cols % 32
    with pytest.raises(tl.TllmError):
        tl.ternarize_pack(np.zeros((2, 192), np.float32))          # cols % group


DIMS = dict(vocab_size=96, hidden_dim=256, intermediate_dim=640, n_layers=2, n_heads=4, n_kv_heads=2,
            max_seq_len=128, head_dim=64, group_size=128, flags=1,
            rope_theta_bits=struct.unpack("<I", struct.pack("<f", 10000.0))[0],
            rms_norm_eps_bits=struct.unpack("<I", struct.pack("<f", 1e-5))[0])


def parse_independently(path):
    """numpy restatement of the file order (reference src/model.cpp:72-212)."""
    raw = np.fromfile(path, dtype=np.uint8)
    hdr = struct.unpack("<15I", raw[:60].tobytes())
    assert hdr[0] == 0x544C4C4D and hdr[1] == 1 and not raw[60:256].any()
    vocab, hidden, inter, layers, heads, kv_heads, _, head_dim = hdr[3:11]
    gs = hdr[12]
    pos = 256 + vocab * hidden * 2
    linears = []

    def take(rows, cols):
        nonlocal pos
        mb, sb = rows * cols // 32 * 4, rows * cols // gs * 2
        nz = raw[pos:pos + mb].view(np.uint32).reshape(rows, cols // 32)
        sg = raw[pos + mb:pos + 2 * mb].view(np.uint32).reshape(rows, cols // 32)
        sc = raw[pos + 2 * mb:pos + 2 * mb + sb].view(np.uint16).reshape(rows, cols // gs)
        pos += 2 * mb + sb
        linears.append((nz, sg, sc))
    for _ in range(layers):
        for rows, cols in ((heads * head_dim, hidden), (kv_heads * head_dim, hidden), (kv_heads * head_dim, hidden),
                           (hidden, heads * head_dim), (inter, hidden), (inter, hidden), (hidden, inter)):
            take(rows, cols)
        pos += 2 * hidden * 2
    pos += hidden * 2
    if hdr[14] & 1:
        take(vocab, hidden)
    else:
        pos += vocab * hidden * 2
    tok = struct.unpack("<Q", raw[pos:pos + 8].tobytes())[0]
    assert pos + 8 + tok == raw.size
    return hdr, linears


def test_model_file_write_open_layout(tmp_path):
    path = str(tmp_path / "tiny.tllm")
    tl.write_synthetic_model(path, seed=11, **DIMS)
    hdr, linears = parse_independently(path)
    mf = tl.ModelFile(path)
    assert mf.header.hidden_dim == 256 and mf.header.n_layers == 2 and mf.header.flags == 1
    assert len(mf.linears) == 7 * 2 + 1 == len(linears)
    pos_pool = 0
    for fl, (nz, sg, sc) in zip(mf.linears, linears):
        assert (fl.rows, fl.cols) == (nz.shape[0], nz.shape[1] * 32)
        assert fl.sign_file - fl.nonzero_file == nz.nbytes and fl.scales_file - fl.sign_file == sg.nbytes
        assert fl.nonzero_pool == pos_pool and fl.nonzero_pool % 256 == 0 and fl.scales_pool % 256 == 0
        pos_pool = fl.scales_pool + (sc.nbytes + 255) // 256 * 256
    assert mf.pool_bytes == pos_pool
    assert [fl.kind for fl in mf.linears[:7]] == list(range(7)) and mf.linears[-1].kind == 7
    # the weights really are ternarised N(0, 0.02^2) draws: about 48 % zeros at factor 0.7, scales near 0.025
    t = synth.unpack_np(*linears[4][:2])
    assert 0.40 < (t == 0).mean() < 0.56
    assert 0.02 < linears[4][2].view(np.float16).astype(np.float64).mean() < 0.03
    mf.close()
    # a second write with the same seed is byte-identical; another seed is not
    path2 = str(tmp_path / "tiny2.tllm")
    tl.write_synthetic_model(path2, seed=11, **DIMS)
    assert open(path, "rb").read() == open(path2, "rb").read()
    tl.write_synthetic_model(path2, seed=12, **DIMS)
    assert open(path, "rb").read() != open(path2, "rb").read()


def test_model_file_rejects_bad_files(tmp_path):
    with pytest.raises(tl.TllmError) as e:
        tl.ModelFile(str(tmp_path / "missing.tllm"))
    assert e.value.code == -8
    bad = tmp_path / "bad.tllm"
    bad.write_bytes(b"\0" * 300)
    with pytest.raises(tl.TllmError) as e:
        tl.ModelFile(str(bad))
    assert e.value.code == -9
    path = str(tmp_path / "t.tllm")
    tl.write_synthetic_model(path, seed=1, **DIMS)
    data = open(path, "rb").read()
    short = tmp_path / "short.tllm"
    short.write_bytes(data[:len(data) // 2])
    with pytest.raises(tl.TllmError) as e:
        tl.ModelFile(str(short))
    assert e.value.code == -8
    with pytest.raises(tl.TllmError):
        tl.write_synthetic_model(path, seed=1, **dict(DIMS, hidden_dim=200))   # not a multiple of the group


def test_model_file_rejects_hostile_headers(tmp_path):
    """Header fields of an untrusted file whose products overflow 32 or 64 bits (heads x head_dim,
    rows x columns, the vocabulary table) must be refused as a bad file, not wrapped into offsets that pass
    the truncation check."""
    import struct
    path = str(tmp_path / "t.tllm")
    tl.write_synthetic_model(path, seed=1, **DIMS)
    good = bytearray(open(path, "rb").read()[:256])
    names = ("magic", "version", "arch", "vocab_size", "hidden_dim", "intermediate_dim", "n_layers", "n_heads",
             "n_kv_heads", "max_seq_len", "head_dim", "rope_theta_bits", "group_size", "rms_norm_eps_bits", "flags")

    def with_fields(**kw):
        h = bytearray(good)
        for k, v in kw.items():
            struct.pack_into("<I", h, 4 * names.index(k), v)
        return bytes(h)

    hostile = [
        dict(n_heads=0x10000, head_dim=0x10000),               # product wraps to 0 in 32 bits
        dict(n_heads=0x8000, head_dim=0x20001),                # product wraps to a small number
        dict(hidden_dim=0xFFFFFFE0),                           # negative as int, pad32 overflows
        dict(vocab_size=0xFFFFFFFF),
        dict(intermediate_dim=0x80000000),
        dict(hidden_dim=1 << 23, intermediate_dim=1 << 23, n_layers=4096),   # each size allowed, a matrix of 2^46 weights
        dict(group_size=0x80000000),
        dict(n_layers=0xFFFFFFFF),
        dict(n_kv_heads=0xFFFFFFFF, head_dim=2),
    ]
    for k, fields in enumerate(hostile):
        f = tmp_path / f"hostile{k}.tllm"
        f.write_bytes(with_fields(**fields) + b"\0" * 4096)
        with pytest.raises(tl.TllmError) as e:
            tl.ModelFile(str(f))
        assert e.value.code == -9, (fields, e.value.code)
    ok = tmp_path / "still_good.tllm"
    ok.write_bytes(open(path, "rb").read())
    tl.ModelFile(str(ok)).close()


@pytest.mark.gpu
def test_model_file_upload_and_sweep(tmp_path, oracle):
    """File -> one device pool -> one plan over every linear of the file -> oracle on the bytes
    parsed independently from the same file."""
    import torch
    path = str(tmp_path / "tiny.tllm")
    tl.write_synthetic_model(path, seed=3, **DIMS)
    _, linears = parse_independently(path)
    mf = tl.ModelFile(path)
    pool = torch.full((mf.pool_bytes,), 0xA5, dtype=torch.uint8, device="cuda")
    mf.upload(pool)
    probs, keep, refs = [], [], []

    class Ptr:  # LinearPlan only needs data_ptr()
        def __init__(self, p):
            self.p = p

        def data_ptr(self):
            return self.p
    for k, (nz, sg, sc) in enumerate(linears):
        pnz, psg, psc, rows, cols = mf.problem(k, pool)
        x = synth.acts_f16(np.random.default_rng(40 + k), 1, cols)
        dx = torch.from_numpy(x).cuda()
        dy = torch.full((1, rows), float("nan"), dtype=torch.float16, device="cuda")
        keep.append((dx, dy))
        probs.append((Ptr(pnz), Ptr(psg), Ptr(psc), dx, dy, rows, cols, 1))
        refs.append(oracle.gemv_f64(nz, sg, sc, x[0].view(np.uint16)))
        got = pool[mf.linears[k].nonzero_pool:mf.linears[k].nonzero_pool + nz.nbytes].cpu().numpy()
        assert np.array_equal(got.view(np.uint32).reshape(nz.shape), nz)          # the upload is byte-exact
    plan = tl.LinearPlan(probs)
    plan.launch()
    torch.cuda.synchronize()
    for k, (ref, (_, dy)) in enumerate(zip(refs, keep)):
        rep = oracle.error_report(dy[0].cpu().numpy().astype(np.float64), ref)
        assert rep["max_rel"] <= 1e-3, (k, rep)
    plan.close()
    mf.close()
