"""The reference's command-line front end (engine/main.cpp), compiled unchanged against include/turbo/*.h by
oracle/Makefile (target ref_cli), links against libturbo12.so with every symbol it uses resolved at start-up."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "oracle", "_ref", "reference_cli")


def test_reference_cli_resolves_every_symbol_it_uses():
    if not os.path.exists(CLI):
        pytest.skip("oracle/_ref/reference_cli not built (needs the reference tree at build time)")
    # LD_BIND_NOW: all of load_model, load_tokenizer, tokenize, generate, forward, sample_greedy, detokenize_one,
    # create_inference_state and the free_* functions are bound before main runs; without arguments the program
    # prints its usage and leaves with 1, touching no GPU
    r = subprocess.run([CLI], capture_output=True, timeout=60, env=dict(os.environ, LD_BIND_NOW="1"))
    assert r.returncode == 1, (r.returncode, r.stderr[-500:])
    assert b"Usage:" in r.stderr and b"--interactive" in r.stderr
    undefined = subprocess.run(["nm", "-D", "--undefined-only", CLI], capture_output=True, timeout=60).stdout.decode()
    for name in ("load_model", "load_tokenizer", "create_inference_state", "generate", "forward", "sample_greedy",
                 "tokenize", "detokenize_one", "free_model", "free_tokenizer", "free_inference_state"):
        assert any(name in line for line in undefined.splitlines()), name
