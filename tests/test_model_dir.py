"""CPU: the loader's host-side directory check (check_model_dir, the first thing load_model does) accepts a
well-formed directory and names what is wrong with a malformed one.  The reference loads whatever it finds and
carries null pointers into the first forward (engine/model.cpp:203-242); here load_model returns nullptr."""
import importlib
import os
import shutil

import numpy as np
import pytest

CFG = dict(n_vocab=96, n_embd=64, n_head=4, n_head_kv=2, n_layer=2, n_ff=128, n_ctx=64,
           rope_theta=500000.0, rms_norm_eps=1e-5)


@pytest.fixture(scope="module")
def good_dir(t12, oracle, tmp_path_factory):
    synth = importlib.import_module("turbo_lossless_amd.synth")
    modelio = importlib.import_module("turbo_lossless_amd.modelio")
    n, ff, kv = CFG["n_embd"], CFG["n_ff"], CFG["n_head_kv"] * (CFG["n_embd"] // CFG["n_head"])
    seed = [10]

    def mk(M, K):
        seed[0] += 1
        p = oracle.pack(synth.weights_llm(M, K, seed[0], p_outlier=2e-2))
        assert p.P > 0
        return p

    layers = [dict(attn_norm=np.ones(n, np.float32), ffn_norm=np.ones(n, np.float32), wq=mk(n, n), wk=mk(kv, n),
                   wv=mk(kv, n), wo=mk(n, n), w_gate=mk(ff, n), w_up=mk(ff, n), w_down=mk(n, ff))
              for _ in range(CFG["n_layer"])]
    path = str(tmp_path_factory.mktemp("good"))
    modelio.write_model_dir(path, CFG, synth.weights_llm(CFG["n_vocab"], n, 5, sigma=1.0, p_outlier=0),
                            np.ones(n, np.float32), mk(CFG["n_vocab"], n), layers)
    return path


@pytest.fixture
def bad_dir(good_dir, tmp_path):
    dst = str(tmp_path / "m")
    shutil.copytree(good_dir, dst)
    return dst


def test_good_directory_passes(t12, good_dir):
    assert t12.check_model_dir(good_dir) == ""


def _rewrite(path, dtype, fn):
    a = np.fromfile(path, dtype)
    fn(a)
    a.tofile(path)


def test_missing_config_and_embeddings(t12, bad_dir, tmp_path):
    assert "config.bin" in t12.check_model_dir(str(tmp_path / "nowhere"))
    os.remove(os.path.join(bad_dir, "tok_embd.bin"))
    assert "tok_embd.bin" in t12.check_model_dir(bad_dir)


@pytest.mark.parametrize("name", ["output_norm.bin", "layer.0.attn_norm.bin", "layer.1.ffn_norm.bin"])
def test_missing_or_short_norm(t12, bad_dir, name):
    p = os.path.join(bad_dir, name)
    np.fromfile(p, np.float32)[:-1].tofile(p)
    assert name in t12.check_model_dir(bad_dir)
    os.remove(p)
    assert name in t12.check_model_dir(bad_dir)


def test_swapped_dims(t12, bad_dir):
    """w_down written with the shape of w_gate: the planes have the right byte count, the role does not fit."""
    p = os.path.join(bad_dir, "layer.0.w_down.dims")
    M, K, P, be = open(p).read().split()
    open(p, "w").write("%s %s %s %s" % (K, M, P, be))
    msg = t12.check_model_dir(bad_dir)
    assert "layer.0.w_down" in msg and "config.bin implies" in msg


def test_tensor_of_another_model(t12, bad_dir):
    p = os.path.join(bad_dir, "layer.1.wq.dims")
    M, K, P, be = open(p).read().split()
    open(p, "w").write("%d %s %s %s" % (int(M) // 2, K, P, be))
    assert "layer.1.wq" in t12.check_model_dir(bad_dir)


def test_malformed_dims_and_base_exp(t12, bad_dir):
    p = os.path.join(bad_dir, "layer.0.wk.dims")
    good = open(p).read()
    open(p, "w").write("sixteen by four")
    assert "malformed" in t12.check_model_dir(bad_dir)
    M, K, P, be = good.split()
    open(p, "w").write("%s %s %s 300" % (M, K, P))
    assert "base_exp" in t12.check_model_dir(bad_dir)
    open(p, "w").write("%s %s %s" % (M, K, P))                 # 4th field optional (engine/model.cpp:38-42)
    assert t12.check_model_dir(bad_dir) == ""
    os.remove(p)
    assert "layer.0.wk.dims" in t12.check_model_dir(bad_dir)


def test_plane_size_mismatch_and_missing_planes(t12, bad_dir):
    p = os.path.join(bad_dir, "layer.0.wv.gr.bin")
    np.fromfile(p, np.uint8)[:-1].tofile(p)
    assert "layer.0.wv" in t12.check_model_dir(bad_dir)
    os.remove(os.path.join(bad_dir, "output_proj.sm.bin"))
    assert "output_proj" in t12.check_model_dir(bad_dir)


def test_escape_list_invariants(t12, bad_dir, good_dir):
    ro = os.path.join(bad_dir, "layer.0.wo.row_off.bin")
    cols = os.path.join(bad_dir, "layer.0.wo.patch_cols.bin")

    def restore():
        for f in ("row_off.bin", "patch_cols.bin", "patch_correct.bin"):
            shutil.copy(os.path.join(good_dir, "layer.0.wo." + f), os.path.join(bad_dir, "layer.0.wo." + f))

    def shift_first(a):
        a[0] = -1
    _rewrite(ro, np.int32, shift_first)
    assert "row_off[0]" in t12.check_model_dir(bad_dir)
    restore()

    def non_monotone(a):
        i = int(np.nonzero(np.diff(a) > 0)[0][0])
        a[i + 1], a[i] = a[i], a[i + 1]
    _rewrite(ro, np.int32, non_monotone)
    msg = t12.check_model_dir(bad_dir)
    assert "monotone" in msg or "row_off[0]" in msg
    restore()

    def last_wrong(a):
        a[-1] += 1
    _rewrite(ro, np.int32, last_wrong)
    assert "row_off[M]" in t12.check_model_dir(bad_dir)
    restore()

    def col_out_of_range(a):
        a[3] = CFG["n_embd"]
    _rewrite(cols, np.int32, col_out_of_range)
    assert "out of range" in t12.check_model_dir(bad_dir)
    restore()

    def col_negative(a):
        a[0] = -5
    _rewrite(cols, np.int32, col_negative)
    assert "out of range" in t12.check_model_dir(bad_dir)
    restore()

    r = np.fromfile(ro, np.int32)
    row = int(np.nonzero(np.diff(r) >= 2)[0][0])               # a row with two escapes: swap them

    def descending(a):
        a[r[row]], a[r[row] + 1] = a[r[row] + 1], a[r[row]]
    _rewrite(cols, np.int32, descending)
    assert "ascend" in t12.check_model_dir(bad_dir)
    restore()

    p = os.path.join(bad_dir, "layer.0.wo.patch_correct.bin")
    np.fromfile(p, np.int16)[:-1].tofile(p)
    assert "escape list files" in t12.check_model_dir(bad_dir)
    restore()
    assert t12.check_model_dir(bad_dir) == ""


def test_rope_scaling_file(t12, bad_dir):
    p = os.path.join(bad_dir, "rope_scaling.bin")
    np.array([8.0, 1.0, 4.0, 8192.0], np.float32).tofile(p)
    assert t12.check_model_dir(bad_dir) == ""
    np.array([8.0, 4.0, 1.0, 8192.0], np.float32).tofile(p)
    assert "rope_scaling" in t12.check_model_dir(bad_dir)
    np.array([8.0, 1.0], np.float32).tofile(p)
    assert "rope_scaling" in t12.check_model_dir(bad_dir)


def test_load_model_refuses_what_the_check_refuses(t12, bad_dir):
    """load_model runs the check before its first GPU call, so the refusal needs no GPU."""
    os.remove(os.path.join(bad_dir, "layer.1.ffn_norm.bin"))
    assert not t12.lib.t12_engine_load(os.fsencode(bad_dir), 0)
