"""The fused-kernel generator: its candidate rule against the candidate lists and
generated file names the reference ships, and the text it emits."""
import itertools
import json
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "tacker_amd", "fusion", "code")
sys.path.insert(0, GEN)

import data  # noqa: E402
import gen_mix  # noqa: E402
import gen_run  # noqa: E402
import kernel_code  # noqa: E402

FIX = json.load(open(os.path.join(ROOT, "tests", "golden", "generator_candidates.json")))
T = data.REFERENCE_KERNEL_INFO


def test_candidate_rule_reproduces_reference_log():
    # fusion/code/log.txt: unreduced (n1, n2, blks) with summed register use
    assert len(FIX["log"]) == 28
    for key, want in FIX["log"].items():
        a, b = key.split()
        got = [[n1, n2, blks, *data.candidate_resources(a, b, (blks, n1, n2), T)]
               for blks, n1, n2 in data.fuse_kernel_info(a, b, T, data.TURING_SM, reduce_gcd=False)]
        assert got == want, key


def test_candidate_rule_reproduces_reference_mix_kernel_info():
    # fusion/code/mix_kernel_info.txt: both kernels as main in turn; the second
    # direction skips ratios the first already produced; registers = max * threads
    assert len(FIX["mix_kernel_info"]) == 42
    for key, want in FIX["mix_kernel_info"].items():
        a, b, main = key.split()
        other = b if main == a else a
        first = [(n1, n2) for _, n1, n2 in data.fuse_kernel_info(a, b, T, data.TURING_SM, reduce_gcd=False)]
        got = []
        for blks, n1, n2 in data.fuse_kernel_info(main, other, T, data.TURING_SM, reduce_gcd=False):
            na, nb = (n1, n2) if main == a else (n2, n1)
            if main == b and (na, nb) in first:
                continue
            _, smem, thr = data.candidate_resources(main, other, (blks, n1, n2), T)
            got.append([na, nb, blks, max(T[a]["register"], T[b]["register"]) * thr, smem, thr])
        assert got == want, key


def test_generated_file_names_match_reference_mix_kernel_directory():
    kernels = sorted(k for k in T if k != "tpacf")
    names = set()
    for a, b in itertools.combinations(kernels, 2):
        names |= set(data.pair_file_names(a, b, T, data.TURING_SM))
    assert sorted(names) == FIX["mix_kernel_files"] and len(names) == 143


def test_cdna4_candidates_fit_one_compute_unit():
    for be in gen_run.BE_KERNELS:
        cands = data.fuse_kernel_info("tzgemm", be)
        assert cands, be
        for c in cands:
            regs, lds, threads = data.candidate_resources("tzgemm", be, c)
            assert regs <= data.CDNA4_CU.registers and lds <= data.CDNA4_CU.shared_memory
            assert threads <= data.CDNA4_CU.thread_slots
        for v in gen_run.pair_candidates(be):
            if v[0] == "wave":
                assert (256 + v[1]) % 64 == 0 and 256 + v[1] <= 768


def test_committed_generated_sources_are_fresh():
    rc = subprocess.run([sys.executable, os.path.join(GEN, "gen_run.py"), "--check"], capture_output=True, text=True)
    assert rc.returncode == 0, rc.stdout + rc.stderr


@pytest.mark.parametrize("be,n_params", [("stencil", 31), ("lbm", 26), ("mriq", 31), ("cp", 27), ("sgemm", 30),
                                         ("fft", 25), ("cutcp", 32)])
def test_emitted_dispatcher_signature(be, n_params):
    # parameter count = the reference dispatcher's (src/mix_kernel/tzgemm_stencil.cu:281-283 31,
    # tzgemm_lbm.cu:352 26, tzgemm_mriq.cu:638 31, tzgemm_cp.cu:994 27, tzgemm_sgemm.cu:303 30, tzgemm_fft.cu:988-996 25, tzgemm_cutcp.cu:345-368 32), order: be first
    text, meta = gen_mix.generate_wg_split(be, 1, 1)
    sig = re.search(r"void (\w+)\(\s*(.*?)\)\s*\{", text, re.S)
    params = [p.strip() for p in sig.group(2).split(",")]
    assert len(params) == n_params and sig.group(1) == f"{be}_tzgemm_mix_wg_1_1"
    names = [p.split()[-1] for p in params]
    assert names[0].startswith(f"{be}0_") and names[-1] == "tzgemm1_ptb_end_block_pos"
    assert names[-15:-9] == ["tzgemm1_A", "tzgemm1_B", "tzgemm1_C", "tzgemm1_NORMAL_M", "tzgemm1_NORMAL_N",
                             "tzgemm1_NORMAL_K"]
    assert names[-9] == "tzgemm1_grid_dimension_x"
    assert names[-3:] == ["tzgemm1_ptb_start_block_pos", "tzgemm1_ptb_iter_block_step", "tzgemm1_ptb_end_block_pos"]
    assert meta["blocksize"] == 256 and meta["group"] == 2
    wave, wmeta = gen_mix.generate_wave_split(be, 256)
    assert "RoleHandoverSync" in wave and "role_wave_done" in wave and wave.count("__syncthreads()") == 1 and wmeta["blocksize"] == 512
    assert f"(int)threadIdx.x - 256" in wave


@pytest.mark.parametrize("name,symbol,n_params", [
    ("tzgemm", "general_ptb_tzgemm", 16), ("stencil", "general_ptb_stencil", 17), ("lbm", "general_ptb_lbm", 12),
    ("mriq", "g_general_ptb_mriq", 17), ("mrif", "general_ptb_mrif", 17), ("cp", "g_general_ptb_cp", 13),
    ("sgemm", "general_ptb_sgemm", 16), ("fft", "g_general_ptb_fft", 11),
    ("cutcp", "general_ptb_cutcp", 18)])
def test_emitted_gptb_kernel_has_the_reference_name_and_parameter_list(name, symbol, n_params):
    # src/gptb_kernel/<name>_kernel.cu: the original kernel's parameters, then 6 dims, start, step, end,
    # thread_base (e.g. stencil_kernel.cu:3-5: 7 + 10; the names are what src/main.cu:108-125 registers)
    text, got_symbol = gen_mix.generate_gptb(name)
    sig = re.search(r"void (\w+)\(\s*(.*?)\)\s*\{", text, re.S)
    names = [p.split()[-1] for p in sig.group(2).split(",")]
    assert sig.group(1) == symbol == got_symbol and len(names) == n_params
    assert names[-10:] == ["grid_dimension_x", "grid_dimension_y", "grid_dimension_z", "block_dimension_x",
                           "block_dimension_y", "block_dimension_z", "ptb_start_block_pos", "ptb_iter_block_step",
                           "ptb_end_block_pos", "thread_base"]
    assert "(int)threadIdx.x - thread_base" in text and "(int)blockIdx.x, ptb_iter_block_step" in text
    files = gen_run.generate()
    assert files[f"gptb_kernel/{name}_kernel.hip"] == text
    assert f'insert("gptb_{name}", (const void *){symbol}, ctx);' in files["gptb_kernel/gptb_kernels.inc"]


def test_gptb_kernels_exist_only_as_generator_output():
    # the library's translation unit includes the generated files and defines no general_ptb_ kernel of
    # its own besides the variant of tzgemm whose workspace is an argument
    text = open(os.path.join(ROOT, "tacker_amd", "csrc", "kernels", "kernels.hip")).read()
    assert '#include "../gptb_kernel/gptb_kernels.inc"' in text
    own = re.findall(r"void (g?_?general_ptb_\w+)\(", text)
    assert own == ["general_ptb_tzgemm_scratch"]


def test_kinfo_emitted_for_every_variant():
    kinfo = json.load(open(os.path.join(ROOT, "tacker_amd", "config", "kinfo-gfx950.json")))
    for be in gen_run.BE_KERNELS:
        base = kinfo[f"tzgemm_{be}"]
        assert {"gridsize", "blocksize", "variant", "block_ratio", "4096"} <= set(base)
        assert f"tzgemm_{be}@{base['variant']}" in kinfo
        assert {"register", "shared_memory", "blocksize", "solo_ptb_blks", "ori_blks"} <= set(kinfo[be])
    assert set(kinfo["throughput_test"]) == {"a", "b"}


def test_best_effort_pairs_are_emitted_in_alphabetical_order_with_kinfo():
    files = gen_run.generate()
    kinfo = json.loads(files["../config/kinfo-gfx950.json"])
    pairs = gen_run.be_pairs()
    names = ["cp", "cutcp", "fft", "lbm", "mrif", "mriq", "sgemm", "stencil"]
    parboil = [(a, b) for i, a in enumerate(names) for b in names[i + 1:]]
    # the Rodinia kernels pair with each other only (src/Creator.cu:554-640,
    # src/mix_kernel/{hot3d_lava,hot3d_nn,hot3d_path,lava_nn,lava_path,nn_path}.cu)
    rodinia = [("hot3d", "lava"), ("hot3d", "nn"), ("hot3d", "path"), ("lava", "nn"), ("lava", "path"), ("nn", "path")]
    assert pairs == sorted(parboil + rodinia) and len(pairs) == 34
    sig = re.search(r"void lava_nn_mix_wg_1_1\(\s*(.*?)\)\s*\{", files["mix_kernel/lava_nn.hip"], re.S)
    params = [q.split() for q in sig.group(1).split(",")]
    assert [q[0] for q in params[:6]] == ["par_str", "dim_str", "box_str*", "FOUR_VECTOR*", "float*", "FOUR_VECTOR*"]  # lava_nn.cu:4-10
    assert len(params) == 15 + 14
    sig = re.search(r"void hot3d_nn_mix_wg_1_1\(\s*(.*?)\)\s*\{", files["mix_kernel/hot3d_nn.hip"], re.S)
    params = [q.split()[-1] for q in sig.group(1).split(",")]
    assert len(params) == 23 + 14 and params[:3] == ["hot3d0_p", "hot3d0_tIn", "hot3d0_tOut"]      # hot3d_nn.cu:4-13
    assert params[23:28] == ["nn1_d_locations", "nn1_d_distances", "nn1_numRecords", "nn1_lat", "nn1_lng"]
    # the fft pairs the reference ships: src/mix_kernel/{cp_fft_3_1,fft_lbm_6_1,fft_mriq_3_2,fft_sgemm_1_4,fft_stencil_5_3}.cu
    sig = re.search(r"void fft_lbm_mix_wg_1_1\(\s*(.*?)\)\s*\{", files["mix_kernel/fft_lbm.hip"], re.S)
    names = [q.split()[-1] for q in sig.group(1).split(",")]
    assert len(names) == 21 and names[0] == "fft0_data" and names[10:12] == ["lbm1_srcGrid", "lbm1_dstGrid"]
    # the four sgemm pairs the reference ships: src/mix_kernel/{cp_sgemm_1_1,lbm_sgemm_1_7,mrif_sgemm_1_4,mriq_sgemm_1_2}.cu
    cp_sgemm = files["mix_kernel/cp_sgemm.hip"]
    sig = re.search(r"void cp_sgemm_mix_wg_1_1\(\s*(.*?)\)\s*\{", cp_sgemm, re.S)
    names = [q.split()[-1] for q in sig.group(1).split(",")]
    assert len(names) == 27 and names[12:18] == ["sgemm1_A", "sgemm1_B", "sgemm1_C", "sgemm1_NORMAL_M", "sgemm1_NORMAL_N",
                                                 "sgemm1_NORMAL_K"]          # cp_sgemm_1_1.cu:163
    assert ("lbm", "mrif") in pairs and ("mrif", "stencil") in pairs   # src/mix_kernel/lbm_mrif_1_3.cu, mrif_stencil_3_2.cu
    assert ("lbm", "mriq") in pairs                       # the pair src/Creator.cu:341-816 also has
    for a, b in pairs:
        text = files[f"mix_kernel/{a}_{b}.hip"]
        for w1, w2 in gen_run.BE_PAIR_SPLITS:
            sym = f"{a}_{b}_mix_wg_{w1}_{w2}"
            assert f"void {sym}(" in text
            entry = kinfo[f"{a}_{b}@wg_{w1}_{w2}"]
            assert entry["group"] == w1 + w2 and entry["blocksize"] == 256
        assert kinfo[f"{a}_{b}"]["variant"] in ("wg_1_1", "wg_1_2", "wg_2_1", "ord_1_1", "ord_1_2", "ord_2_1")
        assert f'insert("{a}_{b}", ' in files["mix_kernel/mix_kernels.inc"]
        # parameter order: the first kernel's list, then the second's
        assert text.index(f"{a}0_grid_dimension_x") < text.index(f"{b}1_grid_dimension_x")
    assert "__shared__" not in files["mix_kernel/lbm_mriq.hip"]        # LDS, where a role uses it, is the role's own


def test_measured_load_ratios_travel_from_profile_ratio_to_the_schedulers_lookup(tmp_path, monkeypatch):
    # profile_ratio.py --apply -> defaults.json -> gen_run.py -> kinfo json -> QosPolicy::blockRatio
    # (src/TaskManager.cu:593-598), on copies of the files, the last step in a fresh process over the
    # recording device layer
    import shutil
    import profile_ratio
    dflt = tmp_path / "defaults.json"
    shutil.copy(os.path.join(GEN, "defaults.json"), dflt)
    monkeypatch.setattr(profile_ratio, "DEFAULTS", str(dflt))
    monkeypatch.setattr(gen_run, "DEFAULTS_PATH", str(dflt))
    ladder = profile_ratio.ladder(132096)
    assert ladder[0] == 129 and ladder[-1] == 132096 and ladder == sorted(set(ladder)) and len(ladder) == 37
    meas = {"stretch": 0.5, "tiles": 1024, "device": "test double",
            "pairs": {"tzgemm_sgemm": {"be_total_blocks": 132096, "be_solo_us": 2000.0,
                                       "by_k": {str(k): {"blocks": 1024 * i, "ratio": float(i) + 0.25}
                                                for i, k in enumerate(profile_ratio.K_LADDER)}}}}
    src = tmp_path / "measured.json"
    src.write_text(json.dumps(meas))
    before = json.loads(dflt.read_text())
    profile_ratio.apply(str(src))
    after = json.loads(dflt.read_text())
    assert after["tzgemm_sgemm"]["ratio_by_k"] == {"128": 0.25, "640": 1.25, "1152": 2.25, "2048": 3.25, "2304": 4.25,
                                                   "4096": 5.25, "4608": 6.25}
    assert after["tzgemm_sgemm"]["block_ratio"] == 5.25 and after["ratio_provenance"]["stretch"] == 0.5
    assert after["tzgemm_stencil"] == before["tzgemm_stencil"]          # pairs that were not measured keep theirs
    with pytest.raises(SystemExit):                                    # a pair the generator does not know
        bad = tmp_path / "bad.json"
        bad.write_text(json.dumps({"stretch": 1.0, "device": "x", "pairs": {"tzgemm_tpacf": {"by_k": {}}}}))
        profile_ratio.apply(str(bad))
    kinfo_text = gen_run.generate()["../config/kinfo-gfx950.json"]
    kinfo = json.loads(kinfo_text)
    assert kinfo["tzgemm_sgemm"]["block_ratio"] == 5.25 and kinfo["tzgemm_sgemm"]["1152"] == 2.25
    kinfo_path = tmp_path / "kinfo.json"
    kinfo_path.write_text(kinfo_text)
    code = ("import sys, ctypes as C; sys.path.insert(0, %r); import tacker_amd as ta; "
            "l = ta.load_library(ta.FAKE_LIB_PATH); assert l.tacker_init(0, %r.encode()) == 0; "
            "l.tacker_qos_block_ratio.restype = C.c_float; "
            "print(l.tacker_qos_block_ratio(b'sgemm', 1152), l.tacker_qos_block_ratio(b'sgemm', 4096), "
            "l.tacker_qos_block_ratio(b'sgemm', 8192), l.tacker_qos_colocated_blocks(0, b'sgemm', 1024, 2304, 132096))"
            % (ROOT, str(kinfo_path)))
    rc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert rc.returncode == 0, rc.stdout + rc.stderr
    got = rc.stdout.strip().splitlines()[-1].split()     # the library's log lines come first
    # a K of the table, the base entry, linear extrapolation from 4096 beyond the table, and the block count
    # Aker mode gives a 1024-tile GEMM of K = 2304: tiles x ratio
    assert [float(v) for v in got[:3]] == [2.25, 5.25, 10.5] and int(got[3]) == int(1024 * 4.25)


def test_a_load_ratio_that_earns_alone_among_its_neighbours_is_taken_as_noise(tmp_path, monkeypatch, capsys):
    # a K whose count cleared the bar while both neighbouring K of the ladder earn nothing is set to 0;
    # positive neighbours keep each other, and so do the ends of the ladder next to a positive K
    import shutil
    import profile_ratio
    dflt = tmp_path / "defaults.json"
    shutil.copy(os.path.join(GEN, "defaults.json"), dflt)
    monkeypatch.setattr(profile_ratio, "DEFAULTS", str(dflt))
    ks = [str(k) for k in profile_ratio.K_LADDER]
    def measured(ratios):
        return {"stretch": 1.0, "min_gain": 0.03, "tiles": 1024, "device": "test double",
                "pairs": {"tzgemm_lbm": {"by_k": {k: {"blocks": int(r * 1024), "ratio": r} for k, r in zip(ks, ratios)},
                                         "whole_kernel": {"serial_us": 100.0, "fused_us": 98.0, "gain": 1.0204}}}}
    src = tmp_path / "m.json"
    src.write_text(json.dumps(measured([0.0, 0.0, 0.0, 1.5, 0.0, 1.5, 0.0])))
    profile_ratio.apply(str(src))
    lbm = json.loads(dflt.read_text())["tzgemm_lbm"]
    assert set(lbm["ratio_by_k"].values()) == {0.0} and lbm["block_ratio"] == 0.0 and lbm["whole_kernel_gain"] == 1.0204
    assert capsys.readouterr().out.count("taken as noise") == 2
    src.write_text(json.dumps(measured([2.0, 0.0, 0.0, 1.5, 1.0, 0.0, 3.0])))
    profile_ratio.apply(str(src))
    lbm = json.loads(dflt.read_text())["tzgemm_lbm"]
    assert [lbm["ratio_by_k"][k] for k in ks] == [0.0, 0.0, 0.0, 1.5, 1.0, 0.0, 0.0]
    src.write_text(json.dumps(measured([2.0, 1.0, 0.0, 0.0, 0.0, 2.5, 3.0])))
    profile_ratio.apply(str(src))
    lbm = json.loads(dflt.read_text())["tzgemm_lbm"]
    assert [lbm["ratio_by_k"][k] for k in ks] == [2.0, 1.0, 0.0, 0.0, 0.0, 2.5, 3.0] and lbm["block_ratio"] == 2.5


def test_profile_tools_import_without_a_gpu_and_know_every_kernel():
    import profile_gptb
    import profile_ratio
    assert set(profile_ratio.PAIRS) == set(gen_run.BE_KERNELS)
    assert profile_gptb.LADDER[-1] == 1.0 and list(profile_gptb.LADDER) == sorted(profile_gptb.LADDER)
    # grids of a million positions and more get a finer run-up (lavaMD: 5832000 positions, 43 ms)
    assert profile_ratio.ladder(5832000)[0] == 5832000 >> 16 and profile_ratio.ladder(528384)[0] == 528384 >> 10
