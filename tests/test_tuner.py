"""The tuner's control flow, failure handling and output formats (the reference's
gemm_tuner.py:34-164 is the model), exercised on the CPU with a stand-in compiler that
"builds" shell scripts; plus what the template must render to."""
import json
import os
import re
import stat
from pathlib import Path

import pytest

from h100_gemm_amd import kernel_configs as kc
from h100_gemm_amd.gemm_tuner import DEFAULT_TEMPLATE, GemmTuner, LATENCY_RE


def fake_compiler(behaviour):
    """compile_command(src, exe) -> argv of a tiny sh program that writes `exe` as a script whose
    behaviour depends on the GROUP constant found in the rendered source."""
    def cmd(src, exe):
        script = f'''
g=$(sed -n 's/.*GROUPM = \\([0-9]*\\);.*/\\1/p' "{src}")
case "{behaviour}-$g" in
  mixed-4)  exit 1 ;;                                                   # compile failure
  mixed-8)  printf '#!/bin/sh\\necho "Shape"\\necho "Correct!"\\necho "Average latency (ms) is %s"\\n' "0.5$g" > "{exe}" ;;
  mixed-16) printf '#!/bin/sh\\necho "Wrong answer! 3 errors!"\\nexit 134\\n' > "{exe}" ;;  # result mismatch -> abort
  mixed-32) printf '#!/bin/sh\\necho "no latency line"\\n' > "{exe}" ;;                # unparsable
  mixed-64) printf '#!/bin/sh\\nsleep 5\\n' > "{exe}" ;;                               # timeout
  *)        printf '#!/bin/sh\\necho "Average latency (ms) is %s"\\n' "1.$g" > "{exe}" ;;
esac
chmod +x "{exe}" 2>/dev/null; exit 0
'''
        return ["sh", "-c", script]
    return cmd


def make_tuner(tmp_path, behaviour="mixed", **kw):
    t = GemmTuner(str(DEFAULT_TEMPLATE), str(tmp_path / "out"), work_dir=str(tmp_path / "work"),
                  compile_command=fake_compiler(behaviour), timeout=1.0, **kw)
    t.param_space = {'KIND': ['ring'], 'BM': [256], 'BN': [256], 'WM': [2], 'WN': [2, 3], 'NS': [4],
                     'SWZ': [1], 'GROUP': [4, 8, 16, 32, 64], 'DTL': [1], 'EPI': [1]}
    return t


def test_failure_classes_score_inf_and_the_sweep_continues(tmp_path):
    t = make_tuner(tmp_path)
    assert not t.is_valid_configuration(dict(KIND='ring', BM=256, BN=256, WM=2, WN=3, NS=4, SWZ=1, GROUP=8, DTL=1, EPI=1))
    best_params, best_runtime, results = t.tune()
    assert len(results) == 5                                  # WN=3 filtered out, five GROUP values run
    by_group = {r['params']['GROUP']: r for r in results}
    assert by_group[8]['success'] and abs(by_group[8]['runtime'] - 0.58) < 1e-9
    for g in (4, 16, 32, 64):                                 # compile fail, bad exit, unparsable, timeout
        assert by_group[g]['success'] is False and by_group[g]['runtime'] is None
    assert best_params['GROUP'] == 8 and best_runtime == by_group[8]['runtime']


def test_output_files_follow_the_reference_formats(tmp_path):
    t = make_tuner(tmp_path, behaviour="allgood")
    best_params, best_runtime, results = t.tune()
    out = tmp_path / "out"
    files = sorted(out.glob("tuning_results_*.json"))
    assert files
    data = json.loads(files[-1].read_text())
    assert set(data) == {'results', 'best_params', 'best_runtime', 'timestamp'}
    assert set(data['results'][0]) == {'params', 'runtime', 'success', 'timestamp'}
    assert data['best_params'] == best_params and data['best_runtime'] == best_runtime
    assert re.fullmatch(r"\d{8}_\d{6}", data['timestamp'])
    summary = (out / "tuning_summary.txt").read_text().splitlines()
    assert summary[0].startswith("Tuning completed at: ")
    assert summary[1] == f"Best runtime: {best_runtime:.4f} ms"
    assert summary[2] == "Best parameters:"
    assert "All successful configurations:" in summary
    runtimes = [float(l.split()[1]) for l in summary if l.startswith("Runtime: ")]
    assert runtimes == sorted(runtimes) and len(runtimes) == 5
    best_src = (out / "best_matmul_mi355x.hip").read_text()
    assert f"GROUPM = {best_params['GROUP']};" in best_src
    # resume: nothing is compiled or run again, the result is the same
    t2 = make_tuner(tmp_path, behaviour="never-called", resume_from=str(files[-1]))
    t2.compile_command = lambda s, e: ["false"]
    bp2, br2, res2 = t2.tune()
    assert bp2 == best_params and br2 == best_runtime and all(r['success'] for r in res2)


def test_no_valid_configuration(tmp_path):
    t = make_tuner(tmp_path)
    t.compile_command = lambda s, e: ["false"]
    best_params, best_runtime, results = t.tune()
    assert best_params is None and best_runtime == float('inf') and len(results) == 5
    assert "Best runtime: inf ms" in (tmp_path / "out" / "tuning_summary.txt").read_text()


def test_template_renders_the_constants_of_a_configuration(tmp_path):
    # the rendering fixture of the reference is matmul_h100_default.cu = its template with the
    # six constants filled in; here: the constants land where the kernels read them
    t = GemmTuner(str(DEFAULT_TEMPLATE), str(tmp_path))
    p = dict(KIND='ring', BM=256, BN=256, WM=2, WN=4, NS=4, SWZ=1, GROUP=16, DTL=1, EPI=1)
    src = t.generate_code(p)
    for line in ["static constexpr int BLOCKM = 256;", "static constexpr int BLOCKN = 256;",
                 "static constexpr int WAVESM = 2;", "static constexpr int WAVESN = 4;",
                 "static constexpr int STAGES = 4;", "static constexpr int GROUPM = 16;",
                 "#define KERNEL_KIND_RING 1", '"r256x256_w2x4_n4_g16"']:
        assert line in src, line
    assert "{{" not in src and "{%" not in src
    p2 = dict(p, KIND='tile', DTL=0, EPI=0)
    assert "#define KERNEL_KIND_TILE 1" in t.generate_code(p2)
    assert t.config_name(p2) == kc.config_name(dict(p2, OCC=1))


def test_default_search_space_is_valid_and_covers_the_shipped_big_kernels():
    t = GemmTuner(output_dir=os.devnull + "_unused") if False else None
    t = GemmTuner.__new__(GemmTuner)
    GemmTuner.__init__(t, str(DEFAULT_TEMPLATE), "/tmp/_tuner_space_check")
    cfgs = t.configurations()
    assert 20 <= len(cfgs) <= 400
    assert all(t.is_valid_configuration(c) for c in cfgs)
    names = {t.config_name(c) for c in cfgs}
    assert "r256x256_w2x2_n4_g8" in names and "t256x256_w2x2_s1_g8_o1_d1_e1" in names
    assert LATENCY_RE.search("Average latency (ms) is 0.8057").group(1) == "0.8057"


def test_the_grid_sweeps_lds_stages_where_the_depth_is_a_parameter(tmp_path):
    """MFMA tile, wave layout and LDS stage count (the reference sweeps BLOCKM and STAGES,
    gemm_tuner.py:17-24): the decode kinds and the small-tile kind appear with several ring
    depths each, every point is a valid configuration with a name of its own, parameters a kind
    ignores do not multiply it, and the template renders every kind."""
    t = GemmTuner(str(DEFAULT_TEMPLATE), str(tmp_path / "out"))
    assert not {"SWZ", "DTL", "EPI"} & set(t.param_space)            # single-valued knobs are not part of the grid
    cfgs = t.configurations()
    names = [t.config_name(c) for c in cfgs]
    assert len(set(names)) == len(names) > 200
    by_kind = {}
    for c in cfgs:
        by_kind.setdefault(c["KIND"], set()).add(c["NS"])
    assert by_kind["stream"] >= {2, 3, 4, 5} and by_kind["decode"] == {3, 4, 5} and by_kind["wavek"] >= {1, 2, 3, 4}
    assert by_kind["tile"] == {4} and by_kind["mfma16"] == {4} and by_kind["ring"] == {4}      # (two-stage kernels: one copy; rings of four)
    for c in cfgs:
        full = dict({"OCC": 1, "SWZ": 1, "DTL": 1, "EPI": 1}, **c)
        if c["KIND"] == "stream":
            full["BN"] = 32
        if c["KIND"] == "wavek" and not c["SHARED"]:
            full.pop("SHARED")
        assert kc.is_valid_config(full), c
    # the library's own decode and small-tile configurations are points of this grid
    for lib in kc.CONFIGS:
        if lib["KIND"] in ("stream", "decode", "wavek"):
            assert kc.config_name(lib) in names, kc.config_name(lib)
    for kind in ("stream", "decode", "wavek"):
        c = next(c for c in cfgs if c["KIND"] == kind and c["NS"] == 3)
        src = t.generate_code(c)
        assert f"#define KERNEL_KIND_{kind.upper()} 1" in src and "static constexpr int STAGES = 3;" in src
        assert f'"{t.config_name(c)}"' in src


def test_cli_keeps_the_kinds_asked_for(tmp_path, monkeypatch, capsys):
    """`--kinds` cuts the grid down to some kernel kinds (the decode shapes are swept over the
    decode and small-tile kinds only); an unknown kind is a usage error."""
    from h100_gemm_amd import gemm_tuner
    seen = {}

    def fake_tune(self, prebuilt=False):
        seen["kinds"] = {c["KIND"] for c in self.configurations()}
        seen["n"] = len(self.configurations())
        seen["args"] = list(self.bench_args)
        seen["bin"] = self.bin_dir
        return None, float("inf"), []

    monkeypatch.setattr(gemm_tuner.GemmTuner, "tune", fake_tune)
    rc = gemm_tuner.main(["--output-dir", str(tmp_path / "o"), "--kinds", "stream,decode", "--shape", "64", "8192", "8192",
                          "--fill", "normal", "--iters", "500", "--bin-dir", str(tmp_path / "b"), "--prebuilt"])
    assert rc == 0 and seen["kinds"] == {"stream", "decode"} and 40 <= seen["n"] <= 60
    assert seen["args"] == ["M", "64", "N", "8192", "K", "8192", "fill", "normal", "iters", "500"]
    assert seen["bin"] == tmp_path / "b"
    with pytest.raises(SystemExit):
        gemm_tuner.main(["--kinds", "wgmma"])
    assert "unknown kind" in capsys.readouterr().err
