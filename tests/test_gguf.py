"""GGUF files: the writer's output is read back by the reader with the
gguf-tools calling interface (CPU), malformed files are refused, and a model
loaded from a file behaves like the one created from the same weights (GPU)."""
import os
import struct

import numpy as np
import pytest

from vkllama_amd import capi, gguf, model as M

CFG = dict(dim=256, n_layers=2, n_heads=4, ffn=352, vocab=640, maxlen=48, eps=1e-5, wtype=8)


@pytest.fixture(scope="module")
def model_file(tmp_path_factory):
    w = M.synth_weights(CFG, seed=9)
    path = str(tmp_path_factory.mktemp("gguf") / "tiny.gguf")
    gguf.write_gguf(path, CFG, w, tokens=["<unk>", "<s>", "</s>", "a", "bc"])
    return path, w


def test_reader_returns_what_the_writer_wrote(model_file):
    path, w = model_file
    g = gguf.read_gguf(path)
    assert g["version"] == 3
    k = g["keys"]
    assert k["llama.attention.head_count"] == (4, CFG["n_heads"])
    assert k["llama.block_count"] == (4, CFG["n_layers"])
    assert k["llama.context_length"] == (4, CFG["maxlen"])
    assert k["llama.attention.layer_norm_rms_epsilon"][0] == 6
    assert abs(k["llama.attention.layer_norm_rms_epsilon"][1] - CFG["eps"]) < 1e-12
    assert k["general.architecture"] == (8, "llama")
    assert k["tokenizer.ggml.tokens"][0] == 9           # arrays are skipped over, not decoded
    assert list(g["tensors"]) == M.tensor_names(CFG["n_layers"])     # file order
    for name, t in g["tensors"].items():
        a = np.ascontiguousarray(w[name])
        assert t["bsize"] == a.nbytes, name
        assert np.array_equal(t["data"], a.view(np.uint8).ravel()), name
        if name.endswith("norm.weight"):
            assert t["type"] == 0 and t["dims"] == [CFG["dim"]]
        else:
            rows, K = M.matrix_shape(CFG, name)
            assert t["type"] == 8 and t["dims"] == [K, rows]


def test_reader_on_a_file_this_repository_did_not_write():
    """tests/golden/handmade_v3.gguf was assembled field by field from the
    published layout of GGUF version 3 (tests/golden/make_gguf_fixture.py, which
    does not use the writer above): the fields the model loader reads
    (models/llama2.h:367-431 of the reference) must come back as spelled out."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "handmade_v3.gguf")
    raw = open(path, "rb").read()
    assert len(raw) < 1024 and raw[:4] == b"GGUF"
    g = gguf.read_gguf(path)
    assert g["version"] == 3
    k = g["keys"]
    assert list(k)[:6] == ["general.architecture", "general.alignment", "llama.context_length",
                           "llama.block_count", "llama.attention.head_count",
                           "llama.attention.layer_norm_rms_epsilon"]          # file order
    assert k["general.architecture"] == (8, "llama")
    assert k["llama.context_length"] == (4, 4096)
    assert k["llama.block_count"] == (4, 32)
    assert k["llama.attention.head_count"] == (4, 32)
    assert k["llama.attention.layer_norm_rms_epsilon"][0] == 6
    assert k["llama.attention.layer_norm_rms_epsilon"][1] == np.float32(1e-5)
    # stepped over correctly: the types and the keys behind them
    assert [k[n][0] for n in ("x.u8", "x.i16", "x.bool", "x.u64", "x.f64")] == [0, 3, 7, 10, 12]
    assert k["tokenizer.ggml.tokens"][0] == 9 and k["x.i32s"][0] == 9
    assert len(k) == 13
    t = g["tensors"]
    assert list(t) == ["output_norm.weight", "blk.0.attn_q.weight", "blk.0.attn_k.weight"]
    n = t["output_norm.weight"]
    assert n["type"] == 0 and n["dims"] == [4] and n["bsize"] == 16
    assert list(n["data"].view(np.float32)) == [1.0, -2.0, 0.5, 3.25]
    q = t["blk.0.attn_q.weight"]
    assert q["type"] == 8 and q["dims"] == [32, 2] and q["bsize"] == 68       # 34 bytes per block of 32
    for row in range(2):
        blk = q["data"][34 * row:34 * row + 34]
        assert blk[:2].view(np.float16)[0] == np.float16(0.25 * (row + 1))
        assert list(blk[2:].view(np.int8)) == [((i * (row + 1) - 16 + 128) % 256) - 128 for i in range(32)]
    # an F16 matrix of 2 rows x 3 columns behind the padding: 1, -0.5, the largest
    # and the smallest normal value, zero, -2.75, as their bit patterns
    h = t["blk.0.attn_k.weight"]
    assert h["type"] == 1 and h["dims"] == [3, 2] and h["bsize"] == 12
    assert h["data"].view(np.uint16).tolist() == [0x3C00, 0xB800, 0x7BFF, 0x0400, 0x0000, 0xC180]


def test_malformed_files_are_refused(model_file, tmp_path):
    path, _ = model_file
    raw = open(path, "rb").read()
    cases = {
        "magic": b"GGUX" + raw[4:],
        "version": raw[:4] + struct.pack("<I", 7) + raw[8:],
        "truncated_header": raw[:200],
        "truncated_data": raw[:len(raw) - 4096],
        "huge_key_count": raw[:16] + struct.pack("<Q", 1 << 40) + raw[24:],
        "empty": b"",
    }
    for name, data in cases.items():
        p = str(tmp_path / (name + ".gguf"))
        open(p, "wb").write(data)
        with pytest.raises(OSError):
            gguf.read_gguf(p)
    with pytest.raises(OSError):
        gguf.read_gguf(str(tmp_path / "missing.gguf"))


@pytest.mark.gpu
def test_model_from_gguf_equals_model_from_weights(model_file):
    path, w = model_file
    prompt = np.array([5, 17, 99, 3], np.uint32)
    a = M.Llama2(CFG, w)
    b = M.Llama2.from_gguf(path)
    assert np.array_equal(a.forward(prompt, 0), b.forward(prompt, 0))
    ia, _, _ = a.generate_greedy(prompt, 16)
    ib, _, _ = b.generate_greedy(prompt, 16)
    assert list(ia) == list(ib)
    a.close(), b.close()
    with pytest.raises(capi.VklError, match=r"\(5\)"):          # NotFound
        M.Llama2.from_gguf(path + ".nope")


@pytest.mark.gpu
def test_infer_cli_on_a_gguf_file(model_file, capsys):
    from vkllama_amd import infer
    path, w = model_file
    assert infer.main([path, "6", "--ids", "5", "17", "99"]) == 0
    out = capsys.readouterr().out
    ids = [int(t) for t in out.split("ids:")[1].split()]
    m = M.Llama2(CFG, w)
    want, _, _ = m.generate_greedy(np.array([5, 17, 99], np.uint32), 6)
    m.close()
    assert ids == [int(t) for t in want]


@pytest.mark.gpu
def test_infer_cli_with_a_sentencepiece_tokenizer(tmp_path, capsys):
    """Text in, text out, the flow of app/llama2_infer.cpp:75-111,178-197: the
    prompt is encoded with a sentencepiece model (BOS first), the generated ids
    are decoded with it.  The tokenizer is trained here on a few sentences
    (64 pieces) and the model's vocabulary has that size."""
    spm = pytest.importorskip("sentencepiece")
    from vkllama_amd import infer
    cfg = dict(CFG, vocab=64)
    w = M.synth_weights(cfg, seed=10)
    path = str(tmp_path / "tiny64.gguf")
    gguf.write_gguf(path, cfg, w, tokens=["<unk>", "<s>", "</s>"])
    corpus = tmp_path / "corpus.txt"
    corpus.write_text("\n".join(["the quick brown fox jumps over the lazy dog",
                                 "hello world this is a test of the tokenizer",
                                 "small models make small talk about the weather today"] * 50))
    spm.SentencePieceTrainer.train(input=str(corpus), model_prefix=str(tmp_path / "tok"), vocab_size=64,
                                   model_type="bpe", bos_id=1, eos_id=2, unk_id=0, minloglevel=2)
    sp = spm.SentencePieceProcessor()
    sp.Load(str(tmp_path / "tok.model"))
    prompt = "hello world"
    assert infer.main([path, "8", "--tokenizer", str(tmp_path / "tok.model"), "--prompt", prompt]) == 0
    lines = capsys.readouterr().out.strip().split("\n")
    ids = [int(t) for t in lines[0].split("ids:")[1].split()]
    m = M.Llama2(cfg, w)
    want, _, _ = m.generate_greedy(np.array([sp.bos_id()] + sp.Encode(prompt), np.uint32), 8)
    m.close()
    assert ids == [int(t) for t in want]
    assert "\n".join(lines[1:]) == sp.Decode(ids)


@pytest.mark.gpu
def test_cpp_llama2_infer_program(model_file):
    """The C++ command-line program (the reference's app/llama2_infer.cpp flow
    on the drop-in classes) prints the same greedy ids."""
    import subprocess
    path, w = model_file
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vkllama_amd", "lib",
                       "llama2_infer")
    r = subprocess.run([exe, path, "6", "5", "17", "99"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-1500:]
    ids = [int(t) for t in r.stdout.split()]
    m = M.Llama2(CFG, w)
    want, _, _ = m.generate_greedy(np.array([5, 17, 99], np.uint32), 6)
    m.close()
    assert ids == [int(t) for t in want]
    bad = subprocess.run([exe, path + ".nope", "2", "1"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 1 and "GGUF" in bad.stderr
