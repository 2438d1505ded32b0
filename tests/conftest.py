"""Shared fixtures: two tiny Qwen3 configurations that differ in every size and option, model
folders with random weights in temporary directories, and a handle on bin/trace_run."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Tiny A: heads*head_dim == hidden, tied head, no window, theta 1e4, eps 1e-6.
TINY_A = dict(architectures=["Qwen3ForCausalLM"], hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0,
              rms_norm_eps=1e-6, max_position_embeddings=128, tie_word_embeddings=True, attention_bias=False,
              use_sliding_window=False, initializer_range=0.02, torch_dtype="bfloat16")
# Tiny B: heads*head_dim (256) != hidden (96), groups of 4, odd vocabulary, untied head, theta 1e6, eps 1e-5.
TINY_B = dict(architectures=["Qwen3ForCausalLM"], hidden_size=96, num_hidden_layers=3, num_attention_heads=8,
              num_key_value_heads=2, head_dim=32, intermediate_size=224, vocab_size=503, rope_theta=1000000.0,
              rms_norm_eps=1e-5, max_position_embeddings=256, tie_word_embeddings=False, attention_bias=False,
              use_sliding_window=False, initializer_range=0.05, torch_dtype="bfloat16")
# Tiny C: B's opposite in the remaining options: a window on layers >= 1, biases on q/k/v, head_dim 48
# (a multiple of 16 that is no power of two), 3 query heads per kv head, 5 layers... kept small.
TINY_C = dict(architectures=["Qwen3ForCausalLM"], hidden_size=80, num_hidden_layers=3, num_attention_heads=6,
              num_key_value_heads=2, head_dim=48, intermediate_size=176, vocab_size=391, rope_theta=50000.0,
              rms_norm_eps=3e-6, max_position_embeddings=512, tie_word_embeddings=False, attention_bias=True,
              use_sliding_window=True, sliding_window=24, max_window_layers=1, initializer_range=0.06,
              torch_dtype="bfloat16")

# Tiny D: head_dim 64 (two 32-dim chunks per head in the matrix-core attention kernels), pairs of query
# heads, three kv heads, theta 5e3, eps 1e-4, tied head.
TINY_D = dict(architectures=["Qwen3ForCausalLM"], hidden_size=72, num_hidden_layers=2, num_attention_heads=6,
              num_key_value_heads=3, head_dim=64, intermediate_size=136, vocab_size=300, rope_theta=5000.0,
              rms_norm_eps=1e-4, max_position_embeddings=320, tie_word_embeddings=True, attention_bias=False,
              use_sliding_window=False, initializer_range=0.04, torch_dtype="bfloat16")

# Tiny E: a window on head_dim 128 (four 32-dim chunks), shorter than the test prompts, on layers >= 1: with
# pages of 16 the bfloat16 engine runs the matrix-core attention kernels over block tables whose first
# pages have been given back.
TINY_E = dict(architectures=["Qwen3ForCausalLM"], hidden_size=88, num_hidden_layers=3, num_attention_heads=4,
              num_key_value_heads=2, head_dim=128, intermediate_size=152, vocab_size=211, rope_theta=20000.0,
              rms_norm_eps=2e-5, max_position_embeddings=640, tie_word_embeddings=False, attention_bias=False,
              use_sliding_window=True, sliding_window=40, max_window_layers=1, initializer_range=0.05,
              torch_dtype="bfloat16")

CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 2), "C": (TINY_C, 5), "D": (TINY_D, 7), "E": (TINY_E, 11)}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """{name: folder} with config.json and model.safetensors (bfloat16 storage)."""
    from ullm_amd.weights.random_init import write_random_model
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = tmp_path_factory.mktemp(f"tiny{name}")
        write_random_model(cfg, str(d), seed=seed)
        out[name] = str(d)
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """{name: (config dict, weights dict)} as the plain implementation reads them."""
    import plain_qwen3 as plain
    return {name: plain.load_model_folder(d) for name, d in model_dirs.items()}


class TraceRun:
    """A running bin/trace_run: send steps, get logits."""

    def __init__(self, model_dir, dtype, out_dir, max_tokens, extra=()):
        self.out_dir = str(out_dir)
        env = dict(os.environ)
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
             "--out", self.out_dir, "--max-tokens", str(max_tokens), *extra],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
        self.step_no = 0

    def step(self, entries, end=(), vocab=None):
        """entries: list of (id, tokens, want). Returns float32 [wanted, vocab] or None."""
        msg = {"step": self.step_no, "entries": [{"id": i, "tokens": list(t), "want": list(w)} for i, t, w in entries],
               "end": list(end)}
        self.proc.stdin.write(json.dumps(msg) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline()
        if line.strip() != f"done {self.step_no}":
            rest = self.proc.stdout.read()
            raise RuntimeError(f"trace_run said {line!r} {rest!r} (exit {self.proc.poll()})")
        path = os.path.join(self.out_dir, f"{self.step_no}.f32")
        self.step_no += 1
        n_want = sum(len(w) for _, _, w in entries)
        if n_want == 0:
            assert not os.path.exists(path)
            return None
        arr = np.fromfile(path, dtype="<f4")
        return arr.reshape(n_want, -1)

    def close(self):
        self.proc.stdin.close()
        rc = self.proc.wait(timeout=60)
        assert rc == 0, f"trace_run exited with {rc}"


@pytest.fixture
def trace_run(tmp_path):
    made = []

    def make(model_dir, dtype, max_tokens, extra=()):
        tr = TraceRun(model_dir, dtype, tmp_path / f"out{len(made)}", max_tokens, extra)
        made.append(tr)
        return tr
    yield make
    for tr in made:
        if tr.proc.poll() is None:
            tr.proc.kill()
