"""The build-time check of the weight-stationary kernels' generated code (csrc/check_ws_isa.py).

The kernels keep a tile in flight in registers that only inline assembly names; compiler-owned
data in those registers ends in a memory fault on the GPU.  These tests feed the checker small
hand-written listings: one clean, and one for each thing it must refuse.
"""
import importlib.util
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
PATH = os.path.join(HERE, "..", "proteinpredictmachinelearning_amd", "csrc", "check_ws_isa.py")
spec = importlib.util.spec_from_file_location("check_ws_isa", PATH)
guard = importlib.util.module_from_spec(spec)
spec.loader.exec_module(guard)

FAST = "_ZN7ppmlhip12_GLOBAL__N_119q8_linear_ws_kernelILi8ELi3ELi8ELi1ELb0EEEvPKhPKfPfiiiiiPhPi"
DUMP = "_ZN7ppmlhip12_GLOBAL__N_119q8_linear_ws_kernelILi8ELi3ELi8ELi1ELb1EEEvPKhPKfPfiiiiiPhPi"
WS64 = "_ZN7ppmlhip12_GLOBAL__N_121q8_linear_ws64_kernelILi4ELi1ELi16ELi0ELb0EEEvPKhPKfPfiiiiiPhPi"


def listing(name, body, owned=256):
    return "\n".join([
        name + ": ; @" + name,
        "\ts_load_dwordx4 s[0:3], s[4:5], 0x0",
        *["\t" + line for line in body],
        "\ts_endpgm",
        "\t.amdhsa_kernel " + name,
        "\t\t.amdhsa_next_free_vgpr %d" % owned,
        "\t.end_amdhsa_kernel",
        ".Lfunc_end0:",
        "",
    ])


CLEAN_BODY = [
    ";;#ASMSTART",
    "global_load_dwordx4 v[240:243], v[2:3], off",
    ";;#ASMEND",
    "v_fma_f32 v239, v1, v2, v3",
    ";;#ASMSTART",
    "s_waitcnt vmcnt(48)",
    "v_mov_b32 v5, v[240]",
    ";;#ASMEND",
]


def run(tmp_path, text):
    f = tmp_path / "k.s"
    f.write_text(text)
    return guard.check(str(f))


def test_clean_listing_passes(tmp_path):
    seen, problems = run(tmp_path, listing(FAST, CLEAN_BODY))
    assert seen == 1 and problems == []


@pytest.mark.parametrize("bad, what", [
    ("v_writelane_b32 v254, s1, 0", "scalar spill"),
    ("v_readlane_b32 s1, v12, 0", "scalar spill"),
    ("scratch_store_dword off, v3, off", "scratch memory"),
    ("v_add_f32_e32 v240, v1, v2", "staging register v240"),
    ("ds_read_b128 v[238:241], v7", "staging register v241"),
])
def test_fast_instance_refused(tmp_path, bad, what):
    seen, problems = run(tmp_path, listing(FAST, CLEAN_BODY + [bad]))
    assert seen == 1 and problems and any(what in p for p in problems)


def test_register_budget_of_the_descriptor(tmp_path):
    _, problems = run(tmp_path, listing(FAST, CLEAN_BODY, owned=240))
    assert len(problems) == 1 and "owns 240 registers" in problems[0]


def test_staging_size_follows_the_kernel_name(tmp_path):
    # 64 staging registers start at v192 in the ws64 kernels; v200 is fine in the 16-register ones
    body = ["v_mov_b32_e32 v200, 0"]
    assert run(tmp_path, listing(FAST, body))[1] == []
    assert len(run(tmp_path, listing(WS64, body))[1]) == 1


def test_diagnostic_instance_may_spill_but_not_stage(tmp_path):
    spills = ["v_writelane_b32 v254, s1, 0", "scratch_store_dword off, v3, off"]
    assert run(tmp_path, listing(DUMP, spills, owned=240))[1] == []
    _, problems = run(tmp_path, listing(DUMP, CLEAN_BODY))
    assert len(problems) == 1 and "staging load" in problems[0]


def test_a_listing_without_kernels_is_an_error(tmp_path):
    seen, problems = run(tmp_path, "\t.text\n")
    assert seen == 0 and problems
