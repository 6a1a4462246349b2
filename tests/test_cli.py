"""The `aker` command line (src/main.cu:227-300 of the reference): argument handling, the lines the
reference's scripts scrape (`fusion/run/run.py:92`: ``[<tag>] <what> took <ms> ms``), and the layout of
recorder_output.txt (src/Recorder.cc:12-44).  CPU: over the recording fake device layer; GPU: the real binary."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCRAPE = re.compile(r'\[(\w+)\] (.+?) took (\d+\.\d+) ms')      # fusion/run/run.py:92


def run(binary, args, cwd):
    path = os.path.join(ROOT, "tacker_amd", "lib", binary)
    if not os.path.exists(path):
        pytest.fail(f"{path} is missing: run `make -C tacker_amd/csrc`")
    env = dict(os.environ, TACKER_QUIET="1")
    return subprocess.run([path] + args, cwd=cwd, env=env, capture_output=True, text=True, timeout=300)


def check_session(p, cwd):
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    out = p.stdout
    assert out.startswith("system: aker, model: vgg16\n")
    assert "Acker Version: " in out and "Compile Timestamp: " in out and "SM num\t\t\t" in out
    assert "[Result] cd1: stencil, cd2: lbm, dnn: vgg16\n" in out                # kinfo "throughput_test"
    assert out.index("[Result] Aker BE task took") < out.index("[Result] Tacker BE task took")
    # the single-number lines are what the scripts' pattern picks up: the fused best-effort pair, once per mode
    assert [(tag, what) for tag, what, _ in SCRAPE.findall(out)] == [("Mix", "BE task1 + task2")] * 2
    assert len(re.findall(r"\[Ori\] BE task1 \+ task2 took [\d.]+ \+ [\d.]+ = [\d.]+ ms to execute\.", out)) == 2
    m = re.search(r"\[Result\] Aker BE task took ([\d.]+) \+ ([\d.]+)\(([\d.]+)\) = ([\d.]+) ms to execute\.", out)
    stage1, stage2, headroom, total = map(float, m.groups())
    assert total == pytest.approx(stage1 + stage2, abs=1e-4) and stage2 >= headroom - 1e-4
    m = re.search(r"\[Result\] Tacker BE task took ([\d.]+) \+ ([\d.]+)\(([\d.]+)\) = ([\d.]+) ms", out)
    stage1, stage2, headroom, total = map(float, m.groups())
    assert stage2 == headroom and total == pytest.approx(stage1 + stage2, abs=1e-4)
    assert len(re.findall(r"\n\[PRE\]lc kernel took \d+\.\d+ ms to execute\.\n", out)) == 2
    # the recorder's table, written at exit
    text = open(os.path.join(cwd, "recorder_output.txt")).read().split("\n")
    assert text[0] == "taskID: 1, taskName: vgg16"
    rows = [l for l in text if l.startswith("    kernelID: ")]
    assert len(rows) == 16                                                       # 13 conv + 3 fc (pooling rides with their inputs)
    for l in rows:
        assert re.fullmatch(r"    kernelID: \d+, kernelName: \w+, execTime: [-+.e\d]+ms", l), l
    assert rows[0].startswith("    kernelID: 100, kernelName: Convolution_conv1_1, execTime: ")
    total_line = text[1 + len(rows)]
    assert re.fullmatch(r"    task running time: [-+.e\d]+ms", total_line) and text[2 + len(rows)] == ""
    times = [float(l.rsplit("execTime: ", 1)[1][:-2]) for l in rows]
    assert float(total_line.split(": ")[1][:-2]) == pytest.approx(sum(times), rel=1e-3)


def test_aker_command_line_over_the_fake_device_layer(tmp_path):
    check_session(run("aker_fake", ["-s", "aker", "-m", "vgg16"], tmp_path), str(tmp_path))
    # long options, device number
    p = run("aker_fake", ["--system", "aker", "--model", "vgg16", "--device", "0"], tmp_path)
    assert p.returncode == 0 and "[Result] Tacker BE task took" in p.stdout


def test_aker_command_line_argument_errors(tmp_path):
    # a missing required option prints the synopsis and returns 0, as the reference's parser branch does
    for args in ([], ["-s", "aker"], ["-m", "vgg16"], ["-s", "aker", "-m"], ["-s", "aker", "-m", "vgg16", "--bogus"]):
        p = run("aker_fake", args, tmp_path)
        assert p.returncode == 0 and p.stdout.startswith("SYNOPSIS") and "system:" not in p.stdout, args
    # an unknown model is a logger.ERROR: exit status 1 (src/main.cu:240-243)
    p = run("aker_fake", ["-s", "aker", "-m", "resnet50"], tmp_path)
    assert p.returncode == 1 and "model not found" in (p.stdout + p.stderr)
    # -c reads a kernel-info file in place of the built-in table
    kinfo = os.path.join(ROOT, "tacker_amd", "config", "kinfo-gfx950.json")
    p = run("aker_fake", ["-s", "aker", "-m", "vgg16", "-c", kinfo], tmp_path)
    assert p.returncode == 0 and "[Result] cd1: stencil, cd2: lbm, dnn: vgg16" in p.stdout
    p = run("aker_fake", ["-s", "aker", "-m", "vgg16", "-c", "/no/such/kinfo.json"], tmp_path)
    assert p.returncode == 1


@pytest.mark.gpu
def test_aker_command_line_on_the_gpu(tmp_path):
    p = run("aker", ["-s", "aker", "-m", "vgg16"], tmp_path)
    check_session(p, str(tmp_path))
    lc = [float(v) for v in re.findall(r"\[PRE\]lc kernel took (\d+\.\d+) ms", p.stdout)]
    assert all(0.1 < v < 50.0 for v in lc), lc                                   # a VGG16 batch-1 query, ms
