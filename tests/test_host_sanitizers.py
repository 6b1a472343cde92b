"""CPU: the host-side parsers of the library (byte-level BPE tables, sentencepiece model reader, and the model
directory check load_model starts with) rebuilt with -fsanitize=address,undefined and run over well-formed,
truncated and corrupted files.  A parser may refuse a file; it may not touch memory outside its buffers."""
import importlib
import io
import os
import random
import shutil
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ENG = os.path.join(ROOT, "turbo-lossless_amd", "csrc", "engine")
SAN = ["-std=c++17", "-g", "-O1", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
       "-fno-omit-frame-pointer"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def build(tmp, with_model_dir):
    exe = os.path.join(tmp, "sanitize_parsers" + ("_dir" if with_model_dir else ""))
    cmd = ["g++", *SAN, "-I" + os.path.join(ROOT, "include"), "-I" + ENG, os.path.join(ROOT, "tests", "sanitize_parsers.cpp"),
           os.path.join(ENG, "tokenizer.cpp"), os.path.join(ENG, "sp_model.cpp")]
    if with_model_dir:
        # model.cpp also holds the GPU half of the loader: its HIP and library calls resolve against the built
        # libraries, none of them runs (check_model_dir is host code only)
        cmd += ["-DWITH_MODEL_DIR", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "turbo-lossless_amd", "csrc"),
                os.path.join(ENG, "model.cpp"), "-L" + os.path.join(ROOT, "turbo-lossless_amd"), "-lturbo12",
                "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath," + os.path.join(ROOT, "turbo-lossless_amd"), "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd + ["-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def run(exe, args):
    r = subprocess.run([exe, *args], capture_output=True, text=True, env=ENV, timeout=600)
    assert r.returncode == 0, (r.stdout[-500:], r.stderr[-4000:])
    return r.stdout.strip().splitlines()[-1]                 # the driver's summary line (the loaders print too)


def mutants(rng, src_dir, out_root, names, n_flip=12):
    """Copies of src_dir with one file truncated (a spread of lengths) or with a few bytes overwritten."""
    dirs = []
    for name in names:
        data = open(os.path.join(src_dir, name), "rb").read()
        cuts = sorted({0, 1, 2, 3, 4, 7, 8, 11, 12, 13, len(data) // 3, len(data) // 2, len(data) - 2, len(data) - 1}
                      | {rng.randrange(len(data)) for _ in range(10)})
        variants = [data[:c] for c in cuts if 0 <= c < len(data)]
        for _ in range(n_flip):
            b = bytearray(data)
            for _ in range(rng.randint(1, 4)):
                b[rng.randrange(len(b))] = rng.choice([0, 1, 0x7F, 0x80, 0xFF, rng.randrange(256)])
            variants.append(bytes(b))
        variants.append(data + b"\xff" * 5)
        for v in variants:
            d = os.path.join(out_root, "m%04d" % len(os.listdir(out_root)))
            shutil.copytree(src_dir, d)
            open(os.path.join(d, name), "wb").write(v)
            dirs.append(d)
    return dirs


def test_tokenizer_parsers_under_sanitizers(t12, tmp_path):
    tf = importlib.import_module(t12.__name__ + ".tokenizer_files")
    rng = random.Random(5)
    exe = build(str(tmp_path), False)
    text = tmp_path / "text.bin"
    text.write_bytes(bytes(rng.choice(b"abcdef \n\xc3\xa9\xff<s>[INST]") for _ in range(3000)))

    # byte-level BPE tables
    alphabet = list(b"abcdef \n")
    syms, merges = [bytes([a]) for a in alphabet], []
    while len(merges) < 40:
        a, b = rng.choice(syms), rng.choice(syms)
        if (a, b) not in merges and len(a + b) < 10:
            merges.append((a, b))
            syms.append(a + b)
    good = tmp_path / "bpe"
    good.mkdir()
    table = tf.bytes_to_unicode()

    def spell(sym):
        return "".join(table[c] for c in sym)
    tf.write_files(str(good), ["<unk>", "<s>", "</s>"] + [spell(s) for s in syms], [(spell(a), spell(b)) for a, b in merges],
                   1, 2, table)
    root = tmp_path / "bpe_mut"
    root.mkdir()
    dirs = [str(good)] + mutants(rng, str(good), str(root), ["vocab.bin", "merges.bin", "byte_encoder.bin"])
    out = run(exe, ["tok", str(text), *dirs])
    assert int(out.split()[1]) >= 1                       # the well-formed one at least

    # sentencepiece model + tokenizer.json
    spm = pytest.importorskip("sentencepiece")
    words = ["".join(rng.choice("abcdefghij") for _ in range(rng.randint(1, 7))) for _ in range(150)] + ["é", "ß"]
    corpus = [" ".join(rng.choice(words) for _ in range(20)) for _ in range(300)]
    buf = io.BytesIO()
    spm.SentencePieceTrainer.train(sentence_iterator=iter(corpus), model_writer=buf, vocab_size=330, model_type="bpe",
                                   normalization_rule_name="identity", character_coverage=1.0, bos_id=1, eos_id=2, unk_id=0,
                                   pad_id=-1, minloglevel=2, byte_fallback=True, user_defined_symbols=["[INST]"])
    sp = tmp_path / "sp"
    sp.mkdir()
    (sp / "tokenizer.model").write_bytes(buf.getvalue())
    (sp / "tokenizer.json").write_text('{"added_tokens": [{"id": 400, "content": "<|x|>", "special": true}, '
                                       '{"id": 401, "content": "a\\"b\\\\u00e9", "special": true}], "model": {"type": "BPE"}}')
    root = tmp_path / "sp_mut"
    root.mkdir()
    dirs = [str(sp)] + mutants(rng, str(sp), str(root), ["tokenizer.model", "tokenizer.json"], n_flip=25)
    out = run(exe, ["tok", str(text), *dirs])
    assert int(out.split()[1]) >= 1


def test_model_directory_check_under_sanitizers(t12, oracle, tmp_path):
    synth = importlib.import_module(t12.__name__ + ".synth")
    modelio = importlib.import_module(t12.__name__ + ".modelio")
    cfg = dict(n_vocab=96, n_embd=64, n_head=4, n_head_kv=2, n_layer=1, n_ff=128, n_ctx=64, rope_theta=500000.0,
               rms_norm_eps=1e-5)
    n, ff, kv = 64, 128, 32
    seed = [20]

    def mk(M, K):
        seed[0] += 1
        return oracle.pack(synth.weights_llm(M, K, seed[0], p_outlier=2e-2))

    layers = [dict(attn_norm=np.ones(n, np.float32), ffn_norm=np.ones(n, np.float32), wq=mk(n, n), wk=mk(kv, n), wv=mk(kv, n),
                   wo=mk(n, n), w_gate=mk(ff, n), w_up=mk(ff, n), w_down=mk(n, ff))]
    good = tmp_path / "model"
    modelio.write_model_dir(str(good), cfg, synth.weights_llm(96, n, 5, sigma=1.0, p_outlier=0), np.ones(n, np.float32),
                            mk(96, n), layers)
    exe = build(str(tmp_path), True)
    rng = random.Random(6)
    root = tmp_path / "mut"
    root.mkdir()
    names = ["config.bin", "layer.0.wo.dims", "layer.0.wo.row_off.bin", "layer.0.wo.patch_cols.bin", "layer.0.wo.sm.bin",
             "output_proj.dims", "output_norm.bin"]
    dirs = [str(good)] + mutants(rng, str(good), str(root), names, n_flip=8)
    out = run(exe, ["dir", *dirs])
    assert int(out.split()[1]) >= 1
