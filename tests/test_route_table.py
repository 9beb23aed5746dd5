"""The route table (which kernel a linear projection runs on) walked on the CPU: launcher and planner read one function
(`linear_route` / `small_kernel`, csrc/route.cpp), so every cell of (layout, format, activation type, rows, size,
flags) must give a plan record that names what the launcher would run, and every route that occurs must have a GPU
parity test.  Reference selection logic: Sources/MetalCompiler/Compiler/MetalPrefillStepBuilder.swift:463-742,
MetalDispatchStepBuilder.swift:640-689, Generator/MetalKernelNameResolver.swift:26-140.  No device is touched."""
import itertools
import os
import re

import pytest

import kat
from conftest import load_package

pkg = load_package()

LAYOUTS = {"blocks": pkg.LAYOUT_STAF_BLOCKS, "planes": pkg.LAYOUT_PLANES, "tile16": pkg.LAYOUT_TILE16}
X_TYPES = {"bf16": pkg.BF16, "f16": pkg.F16, "f32": pkg.F32}
ROWS = [1, 2, 3, 4, 8, 9, 16, 17, 32, 64, 96, 97, 128, 384, 512, 1024, 2048, 4096]
SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336), (1024, 4096), (8192, 2048), (96, 512), (300, 192)]
FLAG_SETS = {"none": 0, "mfma": pkg.FLAG_FORCE_MFMA, "two-step": pkg.FLAG_FORCE_TWO_STEP, "small": pkg.FLAG_FORCE_SMALL_M,
             "generic": pkg.FLAG_FORCE_GENERIC, "stream": pkg.FLAG_FORCE_STREAM}

# what a launcher route must look like in the plan record (regular expression on the '+'-joined device kernels)
PLAN_OF_ROUTE = {
    "two-step": r"^dequant_q\d_g\d+_(bf16|f16|f32)\+hipblaslt_gemm_(bf16|f16|f32)(_x2)?$",
    "stream": r"^qgemm_stream_q\d_g\d+$",
    "fused/wide": r"^(split_f32_bf16x2\+)?qgemm_wide_q\d_g\d+$",
    "fused/tiled": r"^qgemm_mfma_q\d_g\d+$",
    "small-batch/tile16": r"^gemv_tile16_q\d_g\d+$",
    "small-batch/mfma-planes": r"^gemv_mfma_planes_q\d_g\d+$",
    "small-batch/dot-planes": r"^gemv_(rows|planes)_q\d_g\d+$",
    "small-batch/staf-in-place": r"^gemv_staf_q\d_g\d+$",
    "small-batch/generic": r"^gemv_generic$",
    "split-rows/stream": r"^split_f32_bf16x3\+qgemm_stream_q\d_g\d+$",
    "split-rows/tile16": r"^split_f32_bf16x3\+gemv_tile16_q\d_g\d+$",
    "split-rows/mfma-planes": r"^split_f32_bf16x3\+gemv_mfma_planes_q\d_g\d+$",
    "split-rows/dot-planes": r"^split_f32_bf16x3\+gemv_(rows|planes)_q\d_g\d+$",
    "split-rows/staf-in-place": r"^split_f32_bf16x3\+gemv_staf_q\d_g\d+$",
}
# the decode entry point's two-step record is one step
PLAN_OF_ROUTE_DECODE = dict(PLAN_OF_ROUTE, **{"two-step": r"^dequant_q\d_g\d+_f32\+hipblaslt_gemm_f32$"})

# a GPU parity test (file::function) for every route the table can give
PARITY_TEST_OF_ROUTE = {
    "two-step": "test_gpu_two_step.py::test_two_step_seeded_ragged_shapes_and_strides",
    "stream": "test_gpu_gemm_stream.py::test_stream_kernel_against_oracle_and_tiled_kernel",
    "fused/wide": "test_gpu_gemm_wide.py::test_config3_prefill_as_dispatched",
    "fused/tiled": "test_gpu_gemm.py::test_mfma_gemm_exact_small_integers",
    "small-batch/tile16": "test_gpu_tile16.py::test_tile16_llama_shapes_all_batch_sizes",
    "small-batch/mfma-planes": "test_gpu_mfma_planes.py::test_mfma_planes_seeded_shapes",
    "small-batch/dot-planes": "test_gpu_parity.py::test_config1_llama3_8b_layer_shapes",
    "small-batch/staf-in-place": "test_gpu_staf_gemv.py::test_in_place_gemv_formats_and_tails",
    "small-batch/generic": "test_gpu_parity.py::test_other_registered_formats_seeded",
    "split-rows/stream": "test_gpu_gemm_stream.py::test_fp32_rows_ride_on_the_stream_kernel",
    "split-rows/tile16": "test_gpu_split_rows.py::test_f32_rows_full_mantissas",
    "split-rows/mfma-planes": "test_gpu_split_rows.py::test_f32_rows_full_mantissas",
    "split-rows/dot-planes": "test_gpu_split_rows.py::test_f32_rows_full_mantissas",
    "split-rows/staf-in-place": "test_gpu_split_rows.py::test_f32_rows_full_mantissas",
}


def cells():
    for f in pkg.QuantizationFormatRegistry.all_formats():
        for lname, layout in LAYOUTS.items():
            for n, k in SHAPES:
                if k % f.group_size:
                    continue
                if layout != pkg.LAYOUT_STAF_BLOCKS and (k * f.bits) % 32:
                    continue
                if layout == pkg.LAYOUT_TILE16 and not (f.bits == 4 and f.group_size == 64 and k % 128 == 0):
                    continue
                yield f, lname, layout, n, k


def walk(flag_names=("none",)):
    for f, lname, layout, n, k in cells():
        for (xname, xd), m, decode, lib, fname in itertools.product(X_TYPES.items(), ROWS, (False, True), (True, False), flag_names):
            if decode and m > 8:
                continue
            launcher, plan = pkg.probe_route(f, layout, n, k, xd, m, flags=FLAG_SETS[fname], decode_entry=decode, library_available=lib)
            yield (f.bits, f.group_size, lname, n, k, xname, m, decode, lib, fname), launcher, plan


def test_plan_records_name_what_the_launcher_runs_in_every_cell():
    seen = {}
    count = 0
    for cell, launcher, plan in walk():
        count += 1
        assert not launcher.startswith("error"), (cell, launcher)
        table = PLAN_OF_ROUTE_DECODE if cell[7] else PLAN_OF_ROUTE
        assert launcher in table, (cell, launcher, plan)
        assert re.match(table[launcher], plan), (cell, launcher, plan)
        # a context without the dense library never plans or runs the library
        if not cell[8]:
            assert launcher != "two-step" and "hipblaslt" not in plan, (cell, launcher, plan)
        seen.setdefault(launcher, cell)
    assert count > 20000
    # the table is not degenerate: every route occurs somewhere
    assert set(seen) == set(PLAN_OF_ROUTE), sorted(set(PLAN_OF_ROUTE) - set(seen))


def test_forced_routes_are_honoured_or_refused_alike():
    """Selection flags: the launcher either takes the forced route or refuses the call; where it runs, the plan names
    the same kernel."""
    for cell, launcher, plan in walk(("mfma", "two-step", "small", "generic", "stream")):
        fname, decode = cell[9], cell[7]
        if launcher.startswith("error"):
            continue
        table = PLAN_OF_ROUTE_DECODE if decode else PLAN_OF_ROUTE
        assert re.match(table[launcher], plan), (cell, launcher, plan)
        if decode:
            continue
        if fname == "mfma":
            assert launcher.startswith("fused/"), (cell, launcher)
        elif fname == "two-step":
            assert launcher == "two-step", (cell, launcher)
        elif fname == "stream":
            assert launcher == "stream", (cell, launcher)
        elif fname == "generic":
            assert launcher in ("small-batch/generic", "two-step"), (cell, launcher)
        elif fname == "small":
            assert launcher.startswith(("small-batch/", "split-rows/", "two-step")), (cell, launcher)


def test_config_routes():
    """The benchmark configurations land where the measurements say they should."""
    q4 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    P, B = pkg.LAYOUT_PLANES, pkg.LAYOUT_STAF_BLOCKS
    r = lambda *a, **kw: pkg.probe_route(*a, **kw)[0]
    assert r(q4, P, 14336, 4096, pkg.BF16, 1, decode_entry=True) == "small-batch/dot-planes"
    assert r(q4, P, 14336, 4096, pkg.BF16, 8, decode_entry=True) == "small-batch/mfma-planes"
    assert r(q4, P, 4096, 4096, pkg.BF16, 3, decode_entry=True) == "small-batch/dot-planes"       # small matrix: rows kernel
    assert r(q4, P, 14336, 4096, pkg.BF16, 64) == "stream"
    assert r(q4, P, 14336, 4096, pkg.BF16, 128) == "fused/wide"          # 56 column tiles x 4 K parts fill the CUs
    assert r(q4, P, 4096, 14336, pkg.BF16, 128) == "fused/tiled"         # 16 column tiles do not
    assert r(q4, P, 4096, 14336, pkg.BF16, 512) == "fused/wide"
    for layout, xd in ((P, pkg.BF16), (B, pkg.BF16), (P, pkg.F16), (B, pkg.F16), (P, pkg.F32), (B, pkg.F32)):
        assert r(q4, layout, 14336, 4096, xd, 2048) == "fused/wide"
        assert r(q4, layout, 4096, 14336, xd, 2048) == "fused/wide"
        assert r(q4, layout, 14336, 4096, xd, 4096) == "two-step"
        assert r(q4, layout, 14336, 4096, xd, 4096, library_available=False) == "fused/wide"
    assert r(q4, B, 14336, 4096, pkg.BF16, 1, decode_entry=True) == "small-batch/staf-in-place"
    assert r(q4, P, 14336, 4096, pkg.F32, 4, decode_entry=True).startswith("split-rows/")


def test_every_route_has_a_gpu_parity_test():
    here = os.path.dirname(os.path.abspath(__file__))
    assert set(PARITY_TEST_OF_ROUTE) == set(PLAN_OF_ROUTE)
    for route, test_id in PARITY_TEST_OF_ROUTE.items():
        path, func = test_id.split("::")
        text = open(os.path.join(here, path)).read()
        assert re.search(rf"^def {func}\(", text, re.M), (route, test_id)
        assert "pytest.mark.gpu" in text, (route, path)


# ---- two or three projections that share their activations (q+k+v, gate+up): shared_route, csrc/route.cpp -------------
SHARED_SHAPES = [((14336, 14336), 4096), ((4096, 1024, 1024), 4096), ((1024, 256, 256), 1024), ((300, 700), 448), ((5, 17, 130), 256)]
# the device kernel a shared launch's plan record must name
PLAN_OF_SHARED_ROUTE = {
    "shared/stream": r"^qgemm_stream_q\d_g\d+$",
    "shared/mfma-planes": r"^gemv_mfma_planes_q\d_g\d+$",
    "shared/dot-planes": r"^gemv_(rows|planes)_q\d_g\d+$",
    "shared/tile16": r"^gemv_tile16_q\d_g\d+$",
    "shared/staf-in-place": r"^gemv_staf_q\d_g\d+$",
    "shared/wide": r"^(split_f32_bf16x2\+)?qgemm_wide_q\d_g\d+$",
    "split-rows": r"^split_f32_bf16x3\+",          # the rows are split once, then the table is asked again for the bf16 rows
    "steps": r".",                                    # the shared launch in steps: the record is the first projection's
    "separate": r".",                                 # a launch per projection: the record is the first projection's own
}
PARITY_TEST_OF_SHARED_ROUTE = {
    "shared/stream": "test_gpu_gemm_stream.py::test_stream_kernel_shared_launch_equals_separate_launches",
    "shared/mfma-planes": "test_gpu_mfma_planes.py::test_mfma_planes_batched_projections_one_launch",
    "shared/dot-planes": "test_gpu_batched.py::test_batched_llama_projections",
    "shared/tile16": "test_gpu_tile16.py::test_tile16_batched_projections_one_launch",
    "shared/staf-in-place": "test_gpu_staf_gemv.py::test_in_place_batched_projections",
    "shared/wide": "test_gpu_gemm_wide.py::test_shared_launch_of_the_wide_kernel_equals_one_matrix_of_all_rows",
    "split-rows": "test_gpu_split_rows.py::test_batched_projections_other_activation_types",
    "steps": "test_gpu_batched.py::test_batched_equals_separate_launches_on_other_routes",
    "separate": "test_gpu_batched.py::test_batched_equals_separate_launches_on_other_routes",
}


def test_shared_launches_plan_what_the_launcher_runs_in_every_cell():
    """mi355q_batched_qgemm and the shared steps of a plan ask one function what the projections run as; the plan record
    of the step names the kernel of the shared launch wherever there is one."""
    seen, count = {}, 0
    for f in pkg.QuantizationFormatRegistry.all_formats():
        for (lname, layout), (ns, k) in itertools.product(LAYOUTS.items(), SHARED_SHAPES):
            if k % f.group_size or (layout != pkg.LAYOUT_STAF_BLOCKS and (k * f.bits) % 32):
                continue
            if layout == pkg.LAYOUT_TILE16 and not (f.bits == 4 and f.group_size == 64 and k % 128 == 0):
                continue
            for (xname, xd), m, fname in itertools.product(X_TYPES.items(), ROWS, FLAG_SETS):
                launcher, plan = pkg.probe_shared_route(f, layout, ns, k, xd, m, flags=FLAG_SETS[fname])
                cell = (f.bits, f.group_size, lname, ns, k, xname, m, fname)
                count += 1
                assert launcher in PLAN_OF_SHARED_ROUTE, (cell, launcher, plan)
                if plan != "error":                       # contradictory flags: the launcher refuses the call as well
                    assert re.match(PLAN_OF_SHARED_ROUTE[launcher], plan), (cell, launcher, plan)
                if fname == "generic":
                    assert not launcher.startswith("shared/"), (cell, launcher)
                if fname in ("stream", "two-step"):         # forced: the matrices together on the stream kernel, or each on its own
                    assert launcher in (("shared/stream", "separate") if fname == "stream" else ("separate",)), (cell, launcher)
                seen.setdefault(launcher, cell)
    assert count > 10000
    assert set(seen) == set(PLAN_OF_SHARED_ROUTE), sorted(set(PLAN_OF_SHARED_ROUTE) - set(seen))
    # the Llama-3-8B decode launches land where the measurements say they should
    q4 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    r = lambda *a, **kw: pkg.probe_shared_route(*a, **kw)[0]
    assert r(q4, pkg.LAYOUT_PLANES, (14336, 14336), 4096, pkg.BF16, 1) == "shared/dot-planes"
    assert r(q4, pkg.LAYOUT_PLANES, (14336, 14336), 4096, pkg.BF16, 8) == "shared/mfma-planes"
    assert r(q4, pkg.LAYOUT_PLANES, (4096, 1024, 1024), 4096, pkg.BF16, 3) == "shared/dot-planes"
    assert r(q4, pkg.LAYOUT_PLANES, (14336, 14336), 4096, pkg.BF16, 32) == "shared/stream"
    assert r(q4, pkg.LAYOUT_TILE16, (14336, 14336), 4096, pkg.BF16, 16) == "shared/tile16"
    assert r(q4, pkg.LAYOUT_STAF_BLOCKS, (14336, 14336), 4096, pkg.BF16, 1) == "shared/staf-in-place"
    assert r(q4, pkg.LAYOUT_STAF_BLOCKS, (14336, 14336), 4096, pkg.BF16, 8) == "shared/stream"
    # prompts: q+k+v and gate+up on the wide-tile kernel as one launch, up to the rows where the dense library takes over
    assert r(q4, pkg.LAYOUT_PLANES, (4096, 1024, 1024), 4096, pkg.BF16, 512) == "shared/wide"
    assert r(q4, pkg.LAYOUT_PLANES, (14336, 14336), 4096, pkg.BF16, 2048) == "shared/wide"
    assert r(q4, pkg.LAYOUT_STAF_BLOCKS, (4096, 1024, 1024), 4096, pkg.F16, 512) == "shared/wide"
    assert pkg.probe_shared_route(q4, pkg.LAYOUT_PLANES, (4096, 1024, 1024), 4096, pkg.F32, 512) == ("shared/wide", "split_f32_bf16x2+qgemm_wide_q4_g64")


def test_every_shared_route_has_a_gpu_parity_test():
    here = os.path.dirname(os.path.abspath(__file__))
    assert set(PARITY_TEST_OF_SHARED_ROUTE) == set(PLAN_OF_SHARED_ROUTE)
    for route, test_id in PARITY_TEST_OF_SHARED_ROUTE.items():
        path, func = test_id.split("::")
        text = open(os.path.join(here, path)).read()
        assert re.search(rf"^def {func}\(", text, re.M), (route, test_id)
        assert "pytest.mark.gpu" in text, (route, path)
