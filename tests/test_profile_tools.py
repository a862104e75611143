"""profile-stage-hip / profile-gemm-hip: the command lines and the log format of the reference's
profiling front ends (frontend/profile-stage.cc, frontend/profile-gemm.cc, profile/profiler.hh:97-100,
185-186), read back the way py/configuration_opt.py:22-38 reads them."""
import os
import subprocess

import pandas as pd
import pytest

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "glinthawk_amd", "lib")
STAGE = os.path.join(LIB, "profile-stage-hip")
GEMM = os.path.join(LIB, "profile-gemm-hip")


def run(args, timeout=120):
    return subprocess.run(args, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)


def test_command_line_refusals(tmp_path):
    assert os.path.exists(STAGE) and os.path.exists(GEMM), "build the tools with `python -m glinthawk_amd.build`"
    log = str(tmp_path / "x.csv")
    r = run([STAGE, "-", "test-gqa4", "static", "all"])
    assert r.returncode != 0 and "Usage:" in r.stderr
    r = run([STAGE, "-", "test-gqa4", "static", "everything", "4", "10", "0", log])
    assert r.returncode != 0 and "Unknown stage: everything" in r.stderr
    r = run([STAGE, "-", "test-gqa4", "ringbuffer", "all", "4", "10", "0", log])
    assert r.returncode != 0 and "Unknown context name" in r.stderr
    r = run([STAGE, "-", "llama9-1t", "static", "all", "4", "10", "0", log])
    assert r.returncode != 0 and "Unknown model name" in r.stderr
    r = run([STAGE, "-", "test-gqa4", "static", "att", "4", "320", "0", log])          # seq_len is 320
    assert r.returncode != 0 and "Token position out of range" in r.stderr
    r = run([GEMM, "64", "512"])
    assert r.returncode != 0 and "Usage:" in r.stderr
    r = run([GEMM, "64", "0", "512", "0", log])
    assert r.returncode != 0 and "positive" in r.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("ctx", ["static", "paged"])
@pytest.mark.parametrize("stage,text", [("all", "Pre+Att+Post+Cls"), ("all_no_cls", "Pre+Att+Post"), ("pre", "Pre"), ("att", "Att"),
                                        ("post", "Post"), ("cls", "Cls")])
def test_profile_stage_log(tmp_path, ctx, stage, text):
    batch, pos, dur = 5, 100, 0
    # the file name the reference's sweep script gives its logs (tools/profile.bash:24)
    log = tmp_path / f"test-gqa4_{stage}_{ctx}_{pos}_{dur}_{batch}.csv"
    r = run([STAGE, "-", "test-gqa4", ctx, stage, str(batch), str(pos), str(dur), str(log)])
    assert r.returncode == 0, r.stderr
    lines = open(log).read().splitlines()
    assert lines[0] == f"# model='test-gqa4', stage={text}, batch_size={batch}, token_pos={pos}, duration_s={dur}"
    assert lines[1] == "repeat,timestamp_ms,duration_us"
    df = pd.read_csv(log, skiprows=1)
    assert list(df.columns) == ["repeat", "timestamp_ms", "duration_us"] and len(df) >= 1
    assert list(df["repeat"]) == list(range(len(df)))
    assert (df["duration_us"] > 0).all() and (df["timestamp_ms"] > 1.6e12).all()
    # the consumer splits the file name into six fields after protecting "all_no_cls"
    assert len(log.name[:-4].replace("all_no_cls", "all-no-cls").split("_")) == 6


@pytest.mark.gpu
def test_profile_stage_runs_for_the_duration(tmp_path):
    log = tmp_path / "test-gqa4_att_static_200_1_8.csv"
    r = run([STAGE, "-", "test-gqa4", "static", "att", "8", "200", "1", str(log)])
    assert r.returncode == 0, r.stderr
    df = pd.read_csv(log, skiprows=1)
    assert len(df) > 50                                    # a 3-layer toy stage: far more than 50 calls per second
    span_ms = df["timestamp_ms"].iloc[-1] - df["timestamp_ms"].iloc[0]
    assert 800 <= span_ms <= 1500
    assert df["duration_us"].to_numpy()[1:].mean() < 5000


@pytest.mark.gpu
def test_profile_gemm_log(tmp_path):
    log = tmp_path / "gemm.csv"
    r = run([GEMM, "64", "1024", "512", "0", str(log)])
    assert r.returncode == 0, r.stderr
    lines = open(log).read().splitlines()
    assert lines[0] == "# dim1='64', dim2=1024, dim3=512, duration_s=0"
    assert lines[1] == "repeat,timestamp_ms,duration_us"
    df = pd.read_csv(log, skiprows=1)
    assert len(df) >= 1 and (df["duration_us"] > 0).all()
