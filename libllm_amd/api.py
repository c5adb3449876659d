"""The Python entry point, in the manner of the reference's binding (python/libllm/__init__.py):
``Model(config_file, device)``, ``model.name``, ``model.complete(prompt, top_k, top_p,
temperature)`` yielding ``Chunk`` objects with ``.text``.  Beside it, ``generate`` serves batches
of token-id prompts and ``step`` exposes the step function.

Tokenisation is not part of this library: a prompt is a list of token ids, or text that a
``tokenizer.json`` beside the model (read with the ``tokenizers`` package, if installed) or a
byte-level fallback turns into ids.
"""
import codecs
import os
from enum import IntEnum
from typing import Iterable, List, Optional, Sequence, Union

from .cache import PAGE
from .engine import Generator, StepEntry
from .errors import ConfigError, RequestError
from .prompt import ControlToken, plain_prompt
from .config import config_from_dir
from .runtime import load_engine, random_engine
from .sampling import Sampler, SamplingParams


class Device(IntEnum):
    """Same values as the reference (python/libllm/__init__.py:46-49).  There is no CPU path."""
    CPU = 0x0000
    CUDA = 0x0100
    GPU = 0x0100
    AUTO = 0x1f00


def parse_device(device) -> Device:
    """A Device, or its name: cpu, cuda (hip and gpu mean the same) or auto (src/libllm/llm.cc:154-168)."""
    if isinstance(device, str):
        names = {"cpu": Device.CPU, "cuda": Device.CUDA, "hip": Device.CUDA, "gpu": Device.CUDA, "auto": Device.AUTO}
        if device.lower() not in names:
            raise ConfigError("invalid device name: must be one of \"cpu\", \"cuda\" or \"auto\"")
        return names[device.lower()]
    return Device(int(device))


class Chunk:
    """A piece of generated output: its text and the token id behind it."""

    def __init__(self, text: str, token_id: Optional[int] = None) -> None:
        self.text = text
        self.token_id = token_id


class _ByteTokenizer:
    """Fallback when no tokenizer file is present: token id = byte value."""

    def __init__(self, vocab: int, bos: Optional[int]):
        if vocab < 256:
            raise RequestError("text prompts need a tokenizer.json or a vocabulary of at least 256")
        self.bos = bos

    def encode(self, text: str) -> List[int]:
        return list(text.encode("utf-8"))

    def control(self, name: str) -> int:
        raise RequestError("control token %r needs a tokenizer.json beside the model" % name)

    def knows(self, name: str) -> bool:
        return False

    def piece(self, token: int) -> bytes:
        return bytes([token]) if token < 256 else ("<%d>" % token).encode()


class _FileTokenizer:
    def __init__(self, path: str):
        from tokenizers import Tokenizer
        self.tok = Tokenizer.from_file(path)

    def encode(self, text: str) -> List[int]:
        return self.tok.encode(text, add_special_tokens=False).ids

    def control(self, name: str) -> int:
        tid = self.tok.token_to_id(name)
        if tid is None:
            raise RequestError("unknown control token %r" % name)
        return tid

    def knows(self, name: str) -> bool:
        return self.tok.token_to_id(name) is not None

    def piece(self, token: int) -> bytes:
        return self.tok.decode([token], skip_special_tokens=False).encode("utf-8")


class Completion:
    """Iterating yields Chunks until a stop token or the token budget ends the reply."""

    def __init__(self, model: "Model", ids: List[int], params: SamplingParams, max_new_tokens: int,
                 stop_tokens: Optional[Iterable[int]] = None):
        self._model, self._ids, self._params, self._max = model, ids, params, max_new_tokens
        self._stop = stop_tokens

    def __iter__(self):
        decoder = codecs.getincrementaldecoder("utf-8")(errors="replace")
        gen = self._model._generator
        for _, token in gen.stream([self._ids], self._params, self._max, self._stop):
            # one chunk per token; its text is empty while a multi-byte character is incomplete
            yield Chunk(decoder.decode(self._model._tokenizer().piece(token)), token)
        tail = decoder.decode(b"", final=True)
        if tail:
            yield Chunk(tail, None)


class Model:
    def __init__(self, config_file: str, device: Union[Device, str] = Device.AUTO, dtype: str = "bfloat16",
                 max_tokens: int = 8192, max_batch: int = 64, ops=None, use_graphs: bool = True,
                 random_weights: bool = False, seed: int = 0, keep_float32: bool = False,
                 tiled_weights: bool = True, max_prompt_rows: int = 16384) -> None:
        """``config_file``: the model folder, or the config.json inside it.  ``device``: a Device
        or one of "auto", "cuda", "hip", "cpu".  With ``random_weights`` only config.json is read
        and every tensor is drawn from ``seed``.  ``keep_float32``: in bfloat16 mode, matrices
        that the file stores in 32-bit stay float32 instead of becoming bfloat16.
        ``tiled_weights=False``: the matrices are held once, not twice (see ``load_engine``).
        ``max_prompt_rows``: the most rows one prompt step of ``generate`` and ``complete``
        brings (it bounds a step's activations); longer batches of prompts take several steps."""
        if int(parse_device(device)) == int(Device.CPU):
            raise ConfigError("this library has no CPU path; use Device.AUTO or Device.GPU")
        model_dir = os.path.dirname(config_file) if os.path.isfile(config_file) else config_file
        self.model_dir = model_dir
        if random_weights:
            self.engine = random_engine(config_from_dir(model_dir), seed=seed, dtype=dtype,
                                        max_tokens=max_tokens, ops=ops, use_graphs=use_graphs,
                                        tiled_weights=tiled_weights)
        else:
            self.engine = load_engine(model_dir, dtype=dtype, max_tokens=max_tokens, ops=ops,
                                      use_graphs=use_graphs, keep_float32=keep_float32,
                                      tiled_weights=tiled_weights)
        self.config = self.engine.config
        spec = self.engine.model.spec
        self._sampler = Sampler(self.engine.ops, spec.vocab)
        self._generator = Generator(self.engine, self._sampler, spec.stop_tokens, spec.max_position,
                                    self.engine.cache.n_pages, PAGE, max_batch=max_batch,
                                    max_prompt_rows=max_prompt_rows)
        self._tok = None

    @property
    def name(self) -> str:
        return self.engine.model.spec.name

    def is_stop(self, token: int) -> bool:
        """Whether the model's configuration names ``token`` as a stop token (src/libllm/llama.cc:390-392)."""
        return int(token) in self.engine.model.spec.stop_tokens

    @property
    def output_dim(self) -> int:
        """The width of a row of logits (src/libllm/llama.cc:398-400)."""
        return self.engine.vocab

    def _tokenizer(self):
        if self._tok is None:
            path = os.path.join(self.model_dir, "tokenizer.json")
            spec = self.engine.model.spec
            self._tok = _FileTokenizer(path) if os.path.isfile(path) else _ByteTokenizer(spec.vocab, spec.bos_token)
        return self._tok

    def build_prompt(self, messages):
        """The prompt of a conversation (``[{"role", "content"}, ...]``, the last message the
        user's, or the assistant's to be continued): in the architecture's chat format, as the
        reference's model class builds it (src/libllm/llama.cc:406-442), where the tokenizer
        beside the model knows the format's control tokens; else the messages as lines of text."""
        build = getattr(self.config, "build_prompt", None)
        if build is not None:
            blocks = build(messages)
            tok = self._tokenizer()
            if all(tok.knows(b._name) for b in blocks if isinstance(b, ControlToken)):
                return blocks
        return plain_prompt(messages)

    def chat_stop_ids(self) -> List[int]:
        """The ids of the control tokens that end a turn in the architecture's chat format, as
        far as the tokenizer beside the model knows them: stop tokens of a chat's replies, beside
        the model's own."""
        tok = self._tokenizer()
        return [tok.control(name) for name in getattr(self.config, "chat_stop_tokens", ()) if tok.knows(name)]

    def _prepare_prompt(self, prompt) -> List[int]:
        if isinstance(prompt, str):
            return self._tokenizer().encode(prompt)
        if isinstance(prompt, list) and prompt and all(isinstance(t, int) for t in prompt):
            return list(prompt)
        if isinstance(prompt, list):
            ids: List[int] = []
            for block in prompt:
                if isinstance(block, str):
                    ids.extend(self._tokenizer().encode(block))
                elif isinstance(block, ControlToken):
                    ids.append(self._tokenizer().control(block._name))
                elif isinstance(block, int):
                    ids.append(block)
                else:
                    raise NotImplementedError()
            return ids
        raise NotImplementedError()

    def complete(self, prompt: Union[str, List[Union[str, int, ControlToken]]], top_k: int = 50,
                 top_p: float = 0.8, temperature: float = 1.0, max_new_tokens: int = 256,
                 seed: int = 0, stop_ids: Optional[Iterable[int]] = None) -> Completion:
        """Completes the prompt; defaults as the reference's (python/libllm/__init__.py:76-77).
        ``stop_ids`` end the reply beside the model's own stop tokens."""
        ids = self._prepare_prompt(prompt)
        if not ids:
            raise RequestError("the prompt is empty")
        stop = None if stop_ids is None else set(self.engine.model.spec.stop_tokens) | {int(t) for t in stop_ids}
        return Completion(self, ids, SamplingParams(temperature, top_k, top_p, seed), max_new_tokens, stop)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 256,
                 temperature: float = 1.0, top_k: int = 50, top_p: float = 0.8, seed: int = 0,
                 stop_tokens: Optional[Iterable[int]] = None, on_token=None) -> List[List[int]]:
        """Generates for every prompt (token ids); as many batches as the cache needs."""
        params = SamplingParams(temperature, top_k, top_p, seed)
        return self._generator.generate(prompts, params, max_new_tokens, stop_tokens, on_token)

    def step(self, entries: Sequence[StepEntry]):
        """One call of the step function; float32 logits ``[wanted, vocab]`` on the device, in a
        tensor of the caller's own (None if nothing is wanted)."""
        logits = self.engine.step(list(entries))
        return None if logits is None else logits.clone()

    def end(self, requests) -> None:
        self.engine.end(requests)
