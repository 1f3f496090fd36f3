"""Building the kernel libraries (ops/library.py), with a stand-in for the compiler: no GPU and no
hipcc needed."""
import os
import stat

import pytest

from pytriton_llama_amd.ops import library


def _fake_compiler(path, body):
    path.write_text("#!/bin/sh\n" + body)
    path.chmod(path.stat().st_mode | stat.S_IXUSR)
    return str(path)


def _output_of(args_line):
    return 'out=""; while [ $# -gt 0 ]; do if [ "$1" = "-o" ]; then out="$2"; fi; shift; done\n' + args_line


@pytest.mark.timeout(120)
def test_a_compiler_that_says_much_does_not_stop_the_build(tmp_path, monkeypatch, capsys):
    """A compiler that writes megabytes of warnings (more than a pipe holds) still ends, and
    the library it wrote is put in place: nobody reads its messages while it runs, so they
    must not go through a pipe."""
    cc = _fake_compiler(tmp_path / "cc", _output_of(
        'i=0; while [ $i -lt 40000 ]; do echo "gemm.hip:1:1: warning: something about line $i of a long file" >&2; '
        'i=$((i+1)); done\nprintf lib > "$out"\n'))
    monkeypatch.setenv("HIPCC", cc)
    monkeypatch.setattr(library, "_build_dir_cache", str(tmp_path))
    library.build(["norm", "rope"], force=True, verbose=False)
    for n in ("norm", "rope"):
        assert (tmp_path / f"libptl_{n}.so").read_text() == "lib"
    assert not [f for f in os.listdir(tmp_path) if ".tmp" in f]


@pytest.mark.timeout(120)
def test_a_failed_compile_names_the_source_and_shows_the_messages(tmp_path, monkeypatch):
    cc = _fake_compiler(tmp_path / "cc", 'echo "norm.hip:7:3: error: no such thing" >&2\nexit 1\n')
    monkeypatch.setenv("HIPCC", cc)
    monkeypatch.setattr(library, "_build_dir_cache", str(tmp_path))
    with pytest.raises(library.KernelLibraryError) as e:
        library.build(["norm"], force=True, verbose=False)
    assert "norm.hip failed to compile" in str(e.value) and "no such thing" in str(e.value)
    assert not [f for f in os.listdir(tmp_path) if f.startswith("libptl_")]
