"""What the measurement script promises without a GPU: one GPU only, said in one line, exit code 2 otherwise."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu_in_one_line():
    for n in ("2", "8"):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", n, "--steps", "3", "--warmup", "1"],
                           capture_output=True, text=True, cwd=ROOT, timeout=60)
        assert r.returncode == 2
        lines = r.stdout.strip().splitlines()
        assert len(lines) == 1 and "one GPU" in lines[0]


def test_bench_names_every_size_flat():
    """The record's config is flat and short: nothing nested, at most 20 keys."""
    sys.path.insert(0, ROOT)
    import bench
    rec = bench.config_record(bench.LLAMA_1B, 16, 8, 2168.5, 512, 8)
    assert len(rec) <= 20 and all(not isinstance(v, (dict, list, tuple)) for v in rec.values())
    assert rec["layers"] == rec["layers_full_model"] == bench.LLAMA_1B["num_hidden_layers"] == 16
    for key, cfg_key in (("hidden_size", "hidden_size"), ("heads", "num_attention_heads"), ("kv_heads", "num_key_value_heads"),
                         ("head_dim", "head_dim"), ("intermediate_size", "intermediate_size"), ("vocab_size", "vocab_size")):
        assert rec[key] == bench.LLAMA_1B[cfg_key]
    assert rec["global_batch"] == 8 and rec["seq_len"] == 4096 and rec["prompt_len"] == 2048
    # what the benchmark calls the engine's defaults are the engine's defaults
    from nanoinfer_amd.engine.scheduler import EngineConfig
    assert bench.DECODE_RUN == EngineConfig().max_decode_run and bench.ENGINE_CHUNK == EngineConfig().prefill_chunk_size
