"""Runs the C++ test driver of the host layer (tests/host/test_main.cc): the reference-style
build -> lower -> routine tests of the plugin surface (collectors, kernels, Device, MemPool,
Resources).  The `cpu` part needs no GPU; the `gpu` part runs every routine on the AMD device and
checks it against the CPU oracle.  The driver runs once per part (one process on the GPU) and every
case of it is one pytest item, so a red run names the operator."""
import os
import re
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "host", "_build", "rg_host_tests")


def _cases():
    """Case names in the order of main(): (those before `if (mode == "gpu")`, those inside it)."""
    text = open(os.path.join(HERE, "host", "test_main.cc")).read()
    main = text[text.index("int main("):]
    cpu_part, gpu_part = main.split('if (mode == "gpu")', 1)
    find = lambda t: re.findall(r"^\s*RUN\((\w+)\);", t, flags=re.M)
    return find(cpu_part), find(gpu_part)


CPU_CASES, GPU_CASES = _cases()


def _run(mode):
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} not built: run `make -C tests/host` (or __graft_entry__.build())")
    proc = subprocess.run([EXE, mode], capture_output=True, text=True, timeout=300)
    verdicts, section, sections = {}, None, {}
    for line in proc.stdout.splitlines():
        m = re.match(r"\[ (RUN |FAIL| OK ) \] (\w+)", line)
        if m and m.group(1) == "RUN ":
            section = m.group(2)
            sections[section] = []
        elif m:
            verdicts[m.group(2)] = m.group(1).strip()
        elif section:
            sections[section].append(line)
    return {"rc": proc.returncode, "verdicts": verdicts, "sections": sections,
            "tail": proc.stdout[-1500:] + proc.stderr[-1500:]}


@pytest.fixture(scope="module")
def cpu_run():
    return _run("cpu")


@pytest.fixture(scope="module")
def gpu_run():
    return _run("gpu")


def _check(run, case):
    verdict = run["verdicts"].get(case)
    if verdict is None:
        started = case in run["sections"]
        pytest.fail(f"{case}: " + ("started but the driver ended before its verdict" if started else "never started")
                    + f" (exit code {run['rc']})\n" + run["tail"])
    assert verdict == "OK", f"{case} failed:\n" + "\n".join(run["sections"].get(case, []))


@pytest.mark.parametrize("case", CPU_CASES)
def test_host_layer_logic_cpu(cpu_run, case):
    _check(cpu_run, case)


@pytest.mark.gpu
@pytest.mark.parametrize("case", GPU_CASES)
def test_host_layer_routines_on_gpu(gpu_run, case):
    _check(gpu_run, case)
