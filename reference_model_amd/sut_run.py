"""System-under-test module for the reference's conformance runner.

The reference's test runner loads a module given with ``--sut-module`` and expects a class ``TosaSUTRunner`` derived
from its ``TosaTestRunner`` with a ``runTestGraph()`` that returns ``(TosaGraphResult, message)``
(``verif/runner/tosa_test_runner.py:59-170,329-335``; the reference model's own module is
``verif/runner/tosa_refmodel_sut_run.py:21-79``).  This module is that class for the MI355X path:

    tosa_verif_run_tests --sut-module reference_model_amd.sut_run -t TEST_DIR
    tosa_verif_run_tests --sut-module reference_model_amd.sut_run \
        --sut-module-args reference_model_amd.sut_run:precise_mode --sut-module-args reference_model_amd.sut_run:no_fusion

It runs ``tosa_mi355_run --test_desc=<desc.json>``, which writes the result files named in ``desc.json`` beside it
and ends with the graph status as its exit code (0 valid, 1 unpredictable, 2 error), as the reference model does.
The executable computes on the GPU only: without one it ends with status 2 and says so.

Runner arguments (``--sut-module-args reference_model_amd.sut_run:NAME[=VALUE]``):
  precise_mode      fp64 results (and the bounds file when desc.json asks for one), like ``--precise_mode=1``
  no_fusion         one kernel per operator (no RESCALE / CLAMP folded into the producer)
  runner=PATH       another build of the executable
"""
from __future__ import annotations

import os
import subprocess
from enum import IntEnum

try:    # inside the reference's runner
    from runner.tosa_test_runner import TosaTestRunner
except ImportError:    # stand-alone use (this package's own tests): the fields runTestGraph() reads, nothing else

    class TosaTestRunner:    # type: ignore[no-redef]
        class TosaGraphResult(IntEnum):
            TOSA_VALID = 0
            TOSA_UNPREDICTABLE = 1
            TOSA_ERROR = 2
            OTHER_ERROR = 3

        def __init__(self, args, runnerArgs, testDirPath):
            self.args, self.runnerArgs, self.testDirPath = args, runnerArgs, testDirPath
            self.descFile = str(testDirPath / "desc.json")


DEFAULT_RUNNER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tosa_mi355_run")


def parse_runner_args(runner_args):
    """NAME or NAME=VALUE strings -> dict (a bare NAME is a flag)."""
    parsed = {}
    for item in runner_args or []:
        name, sep, value = item.partition("=")
        parsed[name] = value if sep else True
    return parsed


class TosaSUTRunner(TosaTestRunner):
    """Runs one test directory through tosa_mi355_run."""

    def __init__(self, args, runnerArgs, testDirPath):
        super().__init__(args, runnerArgs, testDirPath)
        self.sutArgs = parse_runner_args(runnerArgs)
        self.compliance = False

    def command(self):
        cmd = [str(self.sutArgs.get("runner", DEFAULT_RUNNER)), f"--test_desc={self.descFile}"]
        if self.sutArgs.get("precise_mode") or getattr(self.args, "precise_mode", False) or self.compliance:
            cmd.append("--precise_mode=1")
        if self.sutArgs.get("no_fusion"):
            cmd.append("--no_fusion")
        return cmd

    def runTestGraph(self):
        results = TosaTestRunner.TosaGraphResult
        cmd = self.command()
        try:
            done = subprocess.run(cmd, capture_output=True, text=True, timeout=float(self.sutArgs.get("timeout", 600)))
        except (OSError, subprocess.TimeoutExpired) as e:
            return results.OTHER_ERROR, f"{' '.join(cmd)}: {e}"
        if getattr(self.args, "verbose", False):
            print(done.stdout, done.stderr, sep="")
        by_code = {0: results.TOSA_VALID, 1: results.TOSA_UNPREDICTABLE, 2: results.TOSA_ERROR}
        graph_result = by_code.get(done.returncode, results.OTHER_ERROR)
        return graph_result, (None if graph_result == results.TOSA_VALID else done.stderr)
