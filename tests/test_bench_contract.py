"""bench.py's contract that needs no GPU: one GPU only; for more it says so in one line and exits with 2."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_in_one_line():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
    env = dict(os.environ, WORLD_SIZE="4", RANK="0")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, timeout=120, env=env)
    assert p.returncode == 2 and len(p.stdout.strip().splitlines()) == 1


def test_the_record_names_every_size_flat():
    """`config` of the JSON line is flat and short: its keys are read from the source, where the
    line is put together (no GPU here to run it)."""
    import ast
    src = open(os.path.join(ROOT, "bench.py")).read()
    tree = ast.parse(src)
    configs = [n for n in ast.walk(tree) if isinstance(n, ast.Dict)
               and any(isinstance(k, ast.Constant) and k.value == "layers_full_model" for k in n.keys)]
    assert len(configs) == 1
    keys = [k.value for k in configs[0].keys]
    assert len(keys) <= 20 and {"layers", "layers_full_model", "hidden_size", "intermediate_size", "num_attention_heads",
                                "num_key_value_heads", "head_dim", "vocab_size", "global_batch", "seq_len"} <= set(keys)
    assert all(not isinstance(v, (ast.Dict, ast.List)) for v in configs[0].values)
