"""The HIP library is found by the hash of its sources, and its absence is an error, not a
fallback."""
import os

import pytest

from return_amd.kernels import build


def test_every_source_is_a_compile_unit():
    units = build.compile_units()
    names = [name for _, _, name in units]
    assert len(names) == len(set(names))
    assert {os.path.basename(src) for src, _, _ in units} == {os.path.basename(s) for s in build.sources()}
    assert len(build.sources()) >= 9                      # norms, products, attention, sampling
    for src, defines, _ in units:
        with open(src) as f:
            text = f.read()
        for d in defines:                                 # a variant's define is used in its source
            assert d[2:].split("=")[0] in text


def test_a_missing_compiler_is_an_error(monkeypatch, tmp_path):
    """Nothing built and no hipcc: the kernel set cannot come up, and says why."""
    monkeypatch.setattr(build, "_lib_dirs", lambda: iter([str(tmp_path / "lib")]))
    monkeypatch.setattr(build.shutil, "which", lambda name: None)
    monkeypatch.setattr(build.os.path, "exists", lambda p, real=os.path.exists: False if p.endswith("hipcc") else real(p))
    assert build.find_current() is None
    with pytest.raises(build.BuildError, match="hipcc not found"):
        build.ensure_built()


def test_a_stale_library_is_not_used(monkeypatch, tmp_path):
    d = tmp_path / "lib"
    d.mkdir()
    (d / build.LIB_NAME).write_bytes(b"not a library")
    (d / (build.LIB_NAME + ".hash")).write_text("0" * 64)
    monkeypatch.setattr(build, "_lib_dirs", lambda: iter([str(d)]))
    assert build.find_current() is None                   # the hash of the sources differs
    (d / (build.LIB_NAME + ".hash")).write_text(build.source_hash())
    monkeypatch.setattr(build, "_lib_dirs", lambda: iter([str(d)]))
    assert build.find_current() == str(d / build.LIB_NAME)


def test_two_builds_at_once_do_not_disturb_each_other(monkeypatch, tmp_path):
    """Two first calls in a fresh checkout build at the same time into the same folder: each has
    objects of its own, both end with the library and its stamp in place, nothing else is left.
    (The compiler is stood in for by a function that writes its output file after a while.)"""
    import threading
    import time
    out = tmp_path / "lib"
    monkeypatch.setattr(build, "_lib_dirs", lambda: iter([str(out)]))
    monkeypatch.setattr(build, "_hipcc", lambda: "hipcc")

    def fake_run(cmd, what):
        target = cmd[cmd.index("-o") + 1]
        if "-shared" in cmd:
            objs = [c for c in cmd if c.endswith(".o")]
            missing = [o for o in objs if not os.path.exists(o)]
            if missing:
                raise build.BuildError(f"linking: {len(missing)} objects are gone")
            time.sleep(0.05)
        else:
            time.sleep(0.02)
        with open(target, "w") as f:
            f.write("x")
        return ""

    monkeypatch.setattr(build, "_run", fake_run)
    errors = []

    def one(delay):
        try:
            time.sleep(delay)
            build.build(force=True)
        except Exception as e:                          # noqa: BLE001 (reported below)
            errors.append(e)

    threads = [threading.Thread(target=one, args=(d,)) for d in (0.0, 0.06, 0.12)]    # each starts while the one before links
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert sorted(os.listdir(out)) == [build.LIB_NAME, build.LIB_NAME + ".hash"]
    assert build.find_current() == str(out / build.LIB_NAME)


def test_the_kernel_set_does_not_come_up_without_a_gpu():
    import torch
    from return_amd.kernels.hip_ops import HipOps, KernelError
    with pytest.raises(KernelError, match="GPU"):
        HipOps("cpu")
    if not torch.cuda.is_available():
        with pytest.raises(KernelError, match="no GPU"):
            HipOps("cuda:0")
