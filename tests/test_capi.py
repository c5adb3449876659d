"""The C API (libllm_amd/csrc/capi/llm.h): names, error codes and the JSON manner of the
reference's (src/libllm/llm.h:42-72), called through ctypes in this process and from a C program.
The parts that need no GPU (JSON handles, argument checks, messages of errors) run everywhere."""
import ctypes
import json
import os
import subprocess
import sysconfig

import numpy as np
import pytest

from libllm_amd.hip import build as hip_build
from plain import files, llama, sampling
from tiny import TINY_A, make_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CAPI = os.path.join(ROOT, "libllm_amd", "csrc", "capi")
INVALID_ARG, INSUFFICIENT_BUFFER, ABORTED, EOF = 0x0100, 0x0101, 0x0102, 0x0103


@pytest.fixture(scope="module")
def lib():
    lib = ctypes.CDLL(hip_build.build_capi(force=False, verbose=False))
    lib.llm_get_last_error_message.restype = ctypes.c_char_p
    lib.llm_init()
    return lib


def new_json(lib, text=None):
    j = ctypes.c_void_p()
    assert lib.llm_json_init(ctypes.byref(j)) == 0
    if text is not None:
        assert lib.llm_json_parse(ctypes.byref(j), text.encode()) == 0, lib.llm_get_last_error_message()
    return j


def dump(lib, j, size=1 << 16):
    buf = ctypes.create_string_buffer(size)
    rc = lib.llm_json_dump(ctypes.byref(j), buf, ctypes.c_int64(size))
    return rc, buf.value.decode()


def test_json_handles(lib):
    j = new_json(lib, '{"b": [1, 2.5, "x"],   "a": null}')
    rc, text = dump(lib, j)
    assert rc == 0 and json.loads(text) == {"b": [1, 2.5, "x"], "a": None}
    assert dump(lib, j, size=4)[0] == INSUFFICIENT_BUFFER
    assert b"insufficient" in lib.llm_get_last_error_message()
    assert lib.llm_json_parse(ctypes.byref(j), b"{not json") == ABORTED
    assert b"JSONDecodeError" in lib.llm_get_last_error_message()
    assert dump(lib, j)[0] == 0                       # a failed parse leaves the old value
    assert lib.llm_json_parse(ctypes.byref(j), None) == INVALID_ARG
    assert lib.llm_json_init(None) == INVALID_ARG
    assert lib.llm_json_destroy(ctypes.byref(j)) == 0 and j.value is None


def test_argument_checks_and_load_errors(lib, tmp_path):
    m, c = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(new_json(lib, "{}"))) == INVALID_ARG   # no init
    assert lib.llm_model_init(ctypes.byref(m)) == 0
    assert lib.llm_completion_init(ctypes.byref(c)) == 0
    # an empty model cannot complete or tell its name
    assert lib.llm_model_complete(ctypes.byref(m), ctypes.byref(new_json(lib, "{}")), ctypes.byref(c)) == INVALID_ARG
    assert lib.llm_model_get_info(ctypes.byref(m), ctypes.byref(new_json(lib))) == INVALID_ARG
    assert lib.llm_completion_get_next_chunk(ctypes.byref(c), ctypes.byref(new_json(lib))) == INVALID_ARG
    for kwargs, word in (('{}', b"filename"),
                         ('{"filename": "x", "devise": "cuda"}', b"unexpected key in kwargs: devise"),
                         ('{"filename": "x", "device": "tpu"}', b"invalid device"),
                         ('{"filename": "x", "device": "cpu"}', b"no CPU path"),
                         ('{"filename": "%s", "device": "auto"}' % tmp_path, b"config.json")):
        assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(new_json(lib, kwargs))) == ABORTED
        assert word in lib.llm_get_last_error_message(), lib.llm_get_last_error_message()
    assert lib.llm_model_destroy(ctypes.byref(m)) == 0 and m.value is None
    assert lib.llm_completion_destroy(ctypes.byref(c)) == 0 and c.value is None


@pytest.fixture(scope="module")
def tiny_model(tmp_path_factory):
    path = make_model(tmp_path_factory.mktemp("capi"), TINY_A, seed=23)
    cfg_json, weights = files.read_model_dir(path)
    return path, llama.PlainConfig(cfg_json), weights


@pytest.mark.gpu
def test_completion_in_this_process(lib, tiny_model):
    path, cfg, weights = tiny_model
    prompt = np.random.default_rng(4).integers(3, cfg.vocab, size=11).tolist()
    want = sampling.generate(cfg, weights, prompt, 6, temperature=0.0)
    m, c = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.llm_model_init(ctypes.byref(m)) == 0
    kwargs = new_json(lib, json.dumps({"filename": path, "device": "cuda", "dtype": "float32", "max_tokens": 1024}))
    assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(kwargs)) == 0, lib.llm_get_last_error_message()
    info = new_json(lib)
    assert lib.llm_model_get_info(ctypes.byref(m), ctypes.byref(info)) == 0
    assert json.loads(dump(lib, info)[1])["vocab_size"] == cfg.vocab
    assert lib.llm_completion_init(ctypes.byref(c)) == 0
    bad = new_json(lib, json.dumps({"token_ids": prompt, "top_q": 1}))
    assert lib.llm_model_complete(ctypes.byref(m), ctypes.byref(bad), ctypes.byref(c)) == ABORTED
    assert b"top_q" in lib.llm_get_last_error_message()
    for _ in range(2):                                # a model serves one completion after another
        ask = new_json(lib, json.dumps({"token_ids": prompt, "top_k": 1, "max_new_tokens": 6}))
        assert lib.llm_model_complete(ctypes.byref(m), ctypes.byref(ask), ctypes.byref(c)) == 0
        chunk, got = new_json(lib), []
        while True:
            rc = lib.llm_completion_get_next_chunk(ctypes.byref(c), ctypes.byref(chunk))
            if rc != 0:
                break
            piece = json.loads(dump(lib, chunk)[1])
            assert "text" in piece
            if piece["token_id"] is not None:
                got.append(piece["token_id"])
        assert rc == EOF, lib.llm_get_last_error_message()
        assert got == want
    assert lib.llm_completion_destroy(ctypes.byref(c)) == 0
    assert lib.llm_model_destroy(ctypes.byref(m)) == 0


@pytest.mark.gpu
def test_completion_from_a_c_program(lib, tiny_model, tmp_path):
    path, cfg, weights = tiny_model
    prompt = np.random.default_rng(9).integers(3, cfg.vocab, size=7).tolist()
    want = sampling.generate(cfg, weights, prompt, 5, temperature=0.0)
    so = hip_build.build_capi(force=False, verbose=False)
    exe = str(tmp_path / "capi_driver")
    libdir = sysconfig.get_config_var("LIBDIR")
    subprocess.run(["gcc", "-O1", "-I", CAPI, os.path.join(ROOT, "tests", "capi_driver.c"), "-o", exe, so,
                    "-Wl,-rpath," + os.path.dirname(so), "-Wl,-rpath," + libdir], check=True)
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}     # it finds the package itself
    out = subprocess.run([exe, path, "float32", ", ".join(map(str, prompt)), "5"], cwd=str(tmp_path), env=env,
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = out.stdout.splitlines()
    assert lines[0].startswith("info ") and json.loads(lines[0][5:])["name"]
    got = [json.loads(l[6:])["token_id"] for l in lines if l.startswith("chunk ")]
    got = [t for t in got if t is not None]
    assert got == want
    assert lines[-1] == "end"
