"""The C-ABI library loads without a GPU and exports every symbol include/ppml_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="ppml_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+)?(?:int|void|size_t|char\s*\*|ppml_hip_\w+\s*\*)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_header_symbols_are_exported_and_bound():
    from proteinpredictmachinelearning_amd import cabi

    names = _declared_symbols()
    assert len(names) >= 15, names
    lib = cabi.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ppml_hip.h but not exported"
    assert set(names) == set(cabi.SIGNATURES), set(names) ^ set(cabi.SIGNATURES)
    assert lib.ppml_hip_abi_version() == 1


def test_backend_header_symbols_are_exported_and_bound():
    from proteinpredictmachinelearning_amd import cabi

    names = _declared_symbols("ppml_hip_backend.h")
    assert len(names) >= 18, names
    lib = cabi.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ppml_hip_backend.h but not exported"
    assert set(names) == set(cabi.BACKEND_SIGNATURES), set(names) ^ set(cabi.BACKEND_SIGNATURES)


def test_weights_header_symbols_are_exported_and_bound():
    from proteinpredictmachinelearning_amd import cabi

    text = open(os.path.join(ROOT, "include", "ppml_hip_weights.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(ppml_(?:gguf|int8)_\w+)\s*\(", text)))
    assert len(names) == 14, names
    lib = cabi.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ppml_hip_weights.h but not exported"
    assert set(names) == set(cabi.WEIGHTS_SIGNATURES), set(names) ^ set(cabi.WEIGHTS_SIGNATURES)


def test_host_side_argument_checks_need_no_gpu():
    from proteinpredictmachinelearning_amd import cabi

    lib = cabi.load()
    # null pointers / bad sizes are rejected before any device work (mul_mat_q8_cuda rc table,
    # src/cuda/MulMatQ8Kernel.cu:479-481)
    assert lib.mul_mat_q8_hip(None, None, None, 4, 4, 32, 0, 1, None, None) == 1
    assert b"bad arguments" in lib.ppml_hip_last_error()
    one = ctypes.c_void_p(16)
    assert lib.mul_mat_q8_hip(one, one, one, 4, 4, 33, 0, 1, None, None) == 2
    assert lib.mul_mat_q8_hip(one, one, one, 4, 4, 32, 9, 1, None, None) == 5
    assert lib.quantize_rows_q8_0_hip(one, one, 33, None) == 1
    assert lib.q8_weight_packed_bytes_hip(768, 256) == 24 * 8 * (1024 + 64)
    assert lib.q8_weight_packed_bytes_hip(768, 250) == 0
    assert lib.mul_mat_hip(None, one, one, 1, 1, 1, None, None) == 1
    dims = [4, 3, 1, 1, 5, 2, 1, 1, 4, 5, 1, 1]        # contraction lengths differ
    assert lib.out_prod_hip(one, one, one, *dims, None) == 1


def test_mulmat_stats_switch_and_empty_table_need_no_gpu():
    from proteinpredictmachinelearning_amd import cabi, ops

    lib = cabi.load()
    before = lib.ppml_hip_mulmat_stats_enable(1)
    try:
        assert lib.ppml_hip_mulmat_stats_enable(-1) == 1            # other values only query
        lib.ppml_hip_mulmat_stats_reset()
        assert ops.mulmat_stats_rows() == []
        assert lib.ppml_hip_mulmat_stats(None, 0) == 0
        # refused calls are not counted: the reference records after its own argument checks as well
        assert lib.mul_mat_hip(None, None, None, 1, 1, 1, None, None) == 1
        assert ops.mulmat_stats_rows() == []
    finally:
        lib.ppml_hip_mulmat_stats_enable(before)
    assert ctypes.sizeof(cabi.MulMatStat) == 32 + 4 * 8 + 8


def test_q8_path_and_flag_constants_match_the_header():
    """The Python operator's names for the kernel families and its flag words are the header's enumerators."""
    from proteinpredictmachinelearning_amd import ops

    text = open(os.path.join(ROOT, "include", "ppml_hip.h")).read()
    enums = {name: int(value) for name, value in re.findall(r"\b(PPML_Q8_(?:PATH|FLAG)_\w+)\s*=\s*(\d+)", text)}
    paths = {v: k for k, v in enums.items() if k.startswith("PPML_Q8_PATH_")}
    assert sorted(paths) == sorted(ops.Q8_PATH_NAMES) == [0, 1, 2, 3]
    for value, name in ops.Q8_PATH_NAMES.items():
        assert paths[value] == "PPML_Q8_PATH_" + name.upper().replace("-", "_"), (value, name)
    flag = lambda n: enums["PPML_Q8_FLAG_" + n]
    fl = ops._Q8_PATH_FLAGS
    assert fl["auto"] == 0
    assert fl["weight-stationary"] == flag("NO_LOW_LATENCY")
    assert fl["tiled"] == flag("NO_LOW_LATENCY") | flag("NO_WEIGHT_STATIONARY")
    assert fl["general"] == flag("NO_LOW_LATENCY") | flag("NO_WEIGHT_STATIONARY") | flag("NO_TILED")
    assert (fl["low-latency-8"], fl["low-latency-16"], fl["low-latency-32"]) == (flag("LOW_LATENCY_8"), flag("LOW_LATENCY_16"), flag("LOW_LATENCY_32"))
    assert fl["weight-stationary-column-parts"] == flag("NO_LOW_LATENCY") | flag("COLUMN_PARTS")
    assert fl["weight-stationary-whole"] == flag("NO_LOW_LATENCY") | flag("NO_COLUMN_PARTS")
    # every flag is its own bit (the three-way low-latency field aside), none collides with ReLU or the Q8_1 rule
    singles = [flag(n) for n in ("RELU", "Q8_1_ACTIVATIONS", "NO_LOW_LATENCY", "NO_WEIGHT_STATIONARY", "LOW_LATENCY_8", "LOW_LATENCY_16",
                                 "COLUMN_PARTS", "NO_COLUMN_PARTS", "NO_TILED")]
    assert sorted(singles) == [1 << i for i in range(9)]
