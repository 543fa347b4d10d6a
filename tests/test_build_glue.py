"""The two builds of the library -- the Makefile (shared library for the C, C++ and Python harnesses)
and the crate's build.rs (static archive for the Rust side, in place of
crates/kiln-marlin-gemm/build.rs:1-108) -- must compile the same (source, define) pairs.  Both read
kiln_amd/csrc/objects.list; these tests hold them to it.  CPU only."""
import re
import subprocess
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "kiln_amd" / "csrc"
CRATE = ROOT / "integration" / "kiln-marlin-gemm"


def manifest_entries():
    rows = []
    for line in (CSRC / "objects.list").read_text().splitlines():
        line = line.strip()
        if not line or line.startswith("#"):
            continue
        parts = line.split(":")
        assert 2 <= len(parts) <= 3, line
        rows.append((parts[0], parts[1], parts[2] if len(parts) == 3 else None))
    return rows


def test_manifest_names_existing_sources_and_unique_objects():
    rows = manifest_entries()
    assert len({r[0] for r in rows}) == len(rows)
    for _, src, flag in rows:
        assert (CSRC / src).is_file(), src
        assert flag is None or flag.startswith("-D")
    # every kernel or host source in csrc/ is compiled at least once
    listed = {r[1] for r in rows}
    on_disk = {p.name for p in CSRC.iterdir() if p.suffix in (".hip", ".cpp")}
    assert listed == on_disk, (sorted(on_disk - listed), sorted(listed - on_disk))


def test_makefile_compiles_exactly_the_manifest():
    """`make -n -B` of the shipped library: the compile lines it would run, as (source, defines)."""
    out = subprocess.run(["make", "-C", str(CSRC), "-n", "-B", "../lib/libkiln_marlin_gemm.so"],
                         check=True, capture_output=True, text=True).stdout
    compiled, link_objects = set(), None
    for line in out.splitlines():
        if " -c " in line:
            src = re.search(r"-c (\S+)", line).group(1)
            obj = re.search(r"-o _obj/(\S+)\.o", line).group(1)
            defines = tuple(sorted(re.findall(r"-D\S+", line)))
            compiled.add((obj, src, defines))
            if src.endswith(".hip"):
                assert "--offload-arch=gfx950" in line and "-packed-fp32-ops" in line, line
        elif "-shared" in line:
            link_objects = set(re.findall(r"_obj/(\S+)\.o", line))
    want = {(o, s, (f,) if f else ()) for o, s, f in manifest_entries()}
    assert compiled == want, (sorted(compiled - want), sorted(want - compiled))
    assert link_objects == {o for o, _, _ in manifest_entries()}


def test_build_rs_reads_the_manifest_and_hard_codes_no_source():
    text = (CRATE / "build.rs").read_text()
    assert 'csrc.join("objects.list")' in text
    for _, src, _ in manifest_entries():
        assert src not in text, f"build.rs names {src} itself; the list in objects.list is the only one"
    assert "--offload-arch=" in text and "-packed-fp32-ops" in text and "amdhip64" in text
    # the parse build.rs does, restated: `object:source[:flag]`, '#' comments, blank lines skipped
    assert "split(':')" in text and "starts_with('#')" in text


def test_crate_extern_block_matches_the_header():
    """Every function the crate declares `extern "C"` exists in include/kiln_w4a16.h with the same
    number of arguments, and the library exports it."""
    import ctypes
    header = (ROOT / "include" / "kiln_w4a16.h").read_text()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    rust = (CRATE / "src" / "lib.rs").read_text()
    block = re.search(r'unsafe extern "C" \{(.*?)\n\}', rust, flags=re.S).group(1)
    decls = re.findall(r"fn (\w+)\((.*?)\)", block, flags=re.S)
    assert {"kiln_marlin_w4a16_gemm", "kiln_w4a16_workspace_bytes", "kiln_w4a16_quantize_and_pack",
            "kiln_w4a16_quantize_and_pack_device"} <= {name for name, _ in decls}
    lib = ctypes.CDLL(str(ROOT / "kiln_amd" / "lib" / "libkiln_marlin_gemm.so"))
    for name, args in decls:
        m = re.search(name + r"\s*\((.*?)\)\s*;", header, flags=re.S)
        assert m, f"{name} is not declared in kiln_w4a16.h"
        c_args = [a for a in m.group(1).split(",") if a.strip() and a.strip() != "void"]
        rust_args = [a for a in args.split(",") if a.strip()]
        assert len(c_args) == len(rust_args), name
        assert hasattr(lib, name)
