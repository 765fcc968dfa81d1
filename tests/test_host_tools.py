"""CPU checks of the two host-side tools around the kernels: bench.py's command line and the generator of the four-wave
GEMM kernel's k-loop."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, cwd=ROOT)
    assert p.returncode != 0
    assert "one GPU" in (p.stderr + p.stdout) and "--gpus 1" in (p.stderr + p.stdout)


def test_bench_help_lists_the_contract_flags():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, cwd=ROOT)
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--workload", "--schedule", "--gemm-kernel", "--headline-only", "--calibration-copy"):
        assert flag in p.stdout, flag


def run_generator(tmp_path, opts=None):
    out = tmp_path / "loop.inc"
    env = dict(os.environ)
    env.pop("W4_OPTS", None)
    if opts:
        env["W4_OPTS"] = opts
    subprocess.run([sys.executable, os.path.join(ROOT, "ml_dataflow_amd", "csrc", "matmul", "gen_w4_loop.py"), str(out)], check=True, env=env, cwd=ROOT)
    return out.read_text()


def test_generated_k_loop_defines_what_the_kernel_uses_and_is_reproducible(tmp_path):
    text = run_generator(tmp_path)
    assert text == run_generator(tmp_path)                                     # no dependence on time, hashing order or the environment
    kernel = open(os.path.join(ROOT, "ml_dataflow_amd", "csrc", "matmul", "gemm_w4_kernel.h")).read()
    used = set(re.findall(r"\bW4D?_(?:MULT|LOAD|M|PKC|PKM|OUTPUTS|INPUTS|VP|VQ)_?[A-Z0-9_]*\b", kernel))
    defined = set(re.findall(r"#define (W4D?_[A-Z0-9_]+)", text))
    assert used and used <= defined, sorted(used - defined)
    # per k-tile of a multiplying wave: 16 x 6 accumulator groups, two k-steps -> 192 MFMAs in each of its two loop bodies' steps
    for name in ("W4_MULT_PKC_ASM", "W4_MULT_PKM_ASM"):
        body = text[text.index("#define " + name):]
        body = body[:body.index("\n#define ", 10)] if "\n#define " in body[10:] else body
        assert body.count("v_mfma_f32_16x16x32_bf16") % 192 == 0 and body.count("v_mfma_f32_16x16x32_bf16") > 0
        assert "s_barrier" in body
    # the loading wave moves a whole k-tile per step, 68 chunks of sixteen bytes per lane, behind a window of 60 chunks that
    # the prologue requests; the window that is still in flight at the end lies behind the last k-tile and is only waited for
    load = text[text.index("#define W4_LOAD_PACKED_ASM"):text.index("#define W4_LOAD_GATHER_ASM")]
    loads, writes = load.count("buffer_load_dwordx4"), load.count("ds_write_b128")
    assert loads > 60 and (loads - 60) % 68 == 0, loads
    assert writes == loads - 60, (loads, writes)
    # the four symmetric waves of the 256 x 384 kernel: per step 192 MFMAs and a quarter of the k-tile's 80 chunks per wave (8 of
    # P, 12 of Q) straight into the LDS; the loop body holds two steps, the first tile's prologue a whole k-tile and the
    # first loads of the next (all of Q, `pre` of P); the wait in front of the barrier leaves the twelve newest loads (Q) out
    for name in ("W4D_PKC_PACKED_ASM", "W4D_PKC_GATHER_ASM", "W4D_PKM_PACKED_ASM", "W4D_PKM_GATHER_ASM"):
        body = text[text.index("#define " + name):]
        body = body[:body.index("\n#define ", 10)]
        pre = int(re.search(r"#define W4D_PRE (\d+)", text).group(1))
        assert body.count("v_mfma_f32_16x16x32_bf16") == 2 * 192
        assert body.count("buffer_load_dwordx4") == 2 * 20 + 20 + 12 + pre and body.count(" lds\\n") == body.count("buffer_load_dwordx4")
        assert body.count("s_waitcnt vmcnt(12)") == 2 and body.count("s_barrier") == 3
        assert "ds_write" not in body
        assert ("v_mov_b32" in body) == name.endswith("GATHER_ASM")                # only gathered rows bring new offsets per tile
    # no instruction that writes through the scalar data cache
    assert not re.search(r"\bs_(store|buffer_store|atomic|dcache_wb)", text)


def test_ablation_switches_drop_only_what_they_name(tmp_path):
    full = run_generator(tmp_path)
    no_mfma = run_generator(tmp_path, "abl=nomfma")
    assert "v_mfma" in full and "v_mfma" not in no_mfma
    assert no_mfma.count("buffer_load_dwordx4") == full.count("buffer_load_dwordx4")
    no_loads = run_generator(tmp_path, "abl=noloads+nowrites")
    assert "buffer_load_dwordx4" not in no_loads and "ds_write_b128" not in no_loads
    assert no_loads.count("v_mfma") == full.count("v_mfma")


def test_bench_restates_the_tiling_rule_of_the_kernels():
    """bench.py names the kernel function behind each launch class (for the roofline object's dominant kernel) and its sweep
    workload prints what the rule picks: both restate ragged_n_prefers_384 of gemm_kernel.h and must carry its constants."""
    header = open(os.path.join(ROOT, "ml_dataflow_amd", "csrc", "matmul", "gemm_kernel.h")).read()
    wide = re.search(r"#define WIDE_TILE_COST\(rounds, k_tiles\) \(\(rounds\) \* \(256 \+ 384\) \* \((\d+) \* \(k_tiles\) \+ (\d+)\)\)", header)
    narrow = re.search(r"#define NARROW_TILE_COST\(rounds, k_tiles\) \(\(rounds\) \* \(256 \+ 288\) \* (\d+) \* \(k_tiles\)\)", header)
    assert wide and narrow
    per_byte, per_tile, base = wide.group(1), wide.group(2), narrow.group(1)
    bench = open(os.path.join(ROOT, "bench.py")).read()
    assert bench.count("640 * (%s * kt + %s)" % (per_byte, per_tile)) == 2
    assert bench.count("544 * %s * kt" % base) == 2
    host = open(os.path.join(ROOT, "ml_dataflow_amd", "csrc", "matmul", "amd_matmul.hip")).read()
    assert "WIDE_TILE_COST(wide, k_tiles) < NARROW_TILE_COST(narrow, k_tiles)" in host      # the host's first look uses the macros themselves
