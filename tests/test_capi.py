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
    # generate and step need a loaded model, a result and a place for the count
    n = ctypes.c_int64()
    assert lib.llm_model_generate(ctypes.byref(m), ctypes.byref(new_json(lib, "{}")), ctypes.byref(new_json(lib))) == INVALID_ARG
    assert lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, "{}")), None, ctypes.c_int64(0),
                              ctypes.byref(n)) == INVALID_ARG
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


@pytest.mark.gpu
def test_generate_and_step_from_c(lib, tiny_model):
    """Batches of unequal prompts and the step function through the C API, against the plain
    implementation; a buffer that is too small is refused before anything runs."""
    path, cfg, weights = tiny_model
    rng = np.random.default_rng(12)
    prompts = [rng.integers(3, cfg.vocab, size=k).tolist() for k in (3, 9, 1)]
    m = ctypes.c_void_p()
    assert lib.llm_model_init(ctypes.byref(m)) == 0
    kwargs = new_json(lib, json.dumps({"filename": path, "device": "hip", "dtype": "fp32", "max_tokens": 1024}))
    assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(kwargs)) == 0, lib.llm_get_last_error_message()
    # generate
    result = new_json(lib)
    ask = new_json(lib, json.dumps({"prompts": prompts, "max_new_tokens": 5, "temperature": 0.0}))
    assert lib.llm_model_generate(ctypes.byref(m), ctypes.byref(ask), ctypes.byref(result)) == 0, \
        lib.llm_get_last_error_message()
    got = json.loads(dump(lib, result)[1])["tokens"]
    assert got == [sampling.generate(cfg, weights, p, 5, temperature=0.0) for p in prompts]
    bad = new_json(lib, json.dumps({"prompts": prompts, "beams": 4}))
    assert lib.llm_model_generate(ctypes.byref(m), ctypes.byref(bad), ctypes.byref(result)) == ABORTED
    assert b"beams" in lib.llm_get_last_error_message()
    # step: two prompts at once, then one token each; the shorter request ends first
    lib.llm_model_step.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    n = ctypes.c_int64()
    a, b = prompts[0], prompts[1]
    line = {"entries": [{"id": "a", "tokens": a, "want": [0, len(a) - 1]}, {"id": "b", "tokens": b, "want": [len(b) - 1]}]}
    small = (ctypes.c_float * 8)()
    rc = lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, json.dumps(line))), small, 8, ctypes.byref(n))
    assert rc == INSUFFICIENT_BUFFER and n.value == 3 * cfg.vocab         # nothing ran: the same step goes again
    buf = (ctypes.c_float * (3 * cfg.vocab))()
    rc = lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, json.dumps(line))), buf, 3 * cfg.vocab, ctypes.byref(n))
    assert rc == 0 and n.value == 3, lib.llm_get_last_error_message()
    out = np.ctypeslib.as_array(buf).reshape(3, cfg.vocab).copy()
    la, lb = llama.logits_all(cfg, weights, a), llama.logits_all(cfg, weights, b)
    ref = np.stack([la[0], la[-1], lb[-1]])
    assert np.abs(out - ref).max() < 2e-4 * max(1.0, np.abs(ref).max())
    line = {"entries": [{"id": "a", "tokens": [7], "want": [0]}, {"id": "b", "tokens": [9], "want": []}], "end": ["b"]}
    rc = lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, json.dumps(line))), buf, 3 * cfg.vocab, ctypes.byref(n))
    assert rc == 0 and n.value == 1
    out = np.ctypeslib.as_array(buf)[:cfg.vocab].copy()
    ref = llama.logits_all(cfg, weights, a + [7])[-1]
    assert np.abs(out - ref).max() < 2e-4 * max(1.0, np.abs(ref).max())
    rc = lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, '{"entries": [], "end": ["a"]}')), None, 0, ctypes.byref(n))
    assert rc == 0 and n.value == 0
    rc = lib.llm_model_step(ctypes.byref(m), ctypes.byref(new_json(lib, '{"entries": [], "end": ["a"]}')), None, 0, ctypes.byref(n))
    assert rc == ABORTED                                                   # released twice
    assert lib.llm_model_destroy(ctypes.byref(m)) == 0


@pytest.mark.gpu
def test_random_weights_from_c(lib, tiny_model, tmp_path):
    """A folder with config.json alone and "random_weights": the same seed gives the same model."""
    import shutil
    path, cfg, _ = tiny_model
    shutil.copy(os.path.join(path, "config.json"), tmp_path / "config.json")
    lib.llm_model_step.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    outs = []
    for seed in (3, 3, 4):
        m = ctypes.c_void_p()
        assert lib.llm_model_init(ctypes.byref(m)) == 0
        kwargs = new_json(lib, json.dumps({"filename": str(tmp_path), "random_weights": True, "seed": seed,
                                           "dtype": "float32", "max_tokens": 256}))
        assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(kwargs)) == 0, lib.llm_get_last_error_message()
        # logits, not greedy tokens: a random model with tied embeddings repeats its last token
        buf, n = (ctypes.c_float * cfg.vocab)(), ctypes.c_int64()
        line = new_json(lib, json.dumps({"entries": [{"id": 0, "tokens": [5, 6, 7], "want": [2]}], "end": [0]}))
        assert lib.llm_model_step(ctypes.byref(m), ctypes.byref(line), buf, cfg.vocab, ctypes.byref(n)) == 0
        outs.append(np.ctypeslib.as_array(buf).copy())
        assert lib.llm_model_destroy(ctypes.byref(m)) == 0
    assert np.isfinite(outs[0]).all() and outs[0].std() > 0
    assert np.array_equal(outs[0], outs[1]) and not np.allclose(outs[0], outs[2])
    kwargs = new_json(lib, json.dumps({"filename": str(tmp_path)}))       # without the flag the tensors are missed
    m = ctypes.c_void_p()
    assert lib.llm_model_init(ctypes.byref(m)) == 0
    assert lib.llm_model_load(ctypes.byref(m), ctypes.byref(kwargs)) == ABORTED
    assert lib.llm_model_destroy(ctypes.byref(m)) == 0
