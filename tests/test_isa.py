"""What the compiler made of the update kernel, checked on the gfx950 assembly (no GPU needed).

The kernel's speed hangs on a few properties of the generated code that a source change can lose
without any test of results noticing: the decision record and the by-value scalars must be read with
scalar loads (a vector load of the record in front of the tile's loads, waited for before the
branch, cost 13 % on the mixed-precision step once), the tile's loads must be non-temporal and its
stores streaming buffer stores, and the straight-line tile code must not spill."""
import os
import re
import subprocess

import pytest

from flextrain_amd import build

pytestmark = pytest.mark.timeout(300)


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    """name -> assembly text of every kernel in ft_adam.hip, compiled with the library's flags."""
    out = tmp_path_factory.mktemp("isa") / "ft_adam.s"
    flags = [f for f in build.HIPCC_FLAGS if f != "-fPIC"]
    cmd = [build.hipcc(), *flags, "-I", build.INCLUDE, "-I", build.CSRC, "--cuda-device-only", "-S",
           os.path.join(build.CSRC, "ft_adam.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    text = out.read_text()
    found = {}
    for match in re.finditer(r"^(_ZN3ftk\w+):.*?\n(.*?)^\.Lfunc_end\d+:", text, re.S | re.M):
        found[match.group(1)] = match.group(2)
    assert found
    return found


def _tile_variants(kernels):
    pattern = re.compile(r"adam_tile_kernelILi(\w+)ELi(\w+)ELb([01])ELb([01])E")
    for name, body in kernels.items():
        m = pattern.search(name)
        if m:
            yield name, m.group(1), m.group(2), m.group(3) == "1", m.group(4) == "1", body


def test_every_tile_kernel_variant_is_there(kernels):
    variants = {(g, h, c, y) for _, g, h, c, y, _ in _tile_variants(kernels)}
    assert len(variants) == 3 * 3 * 2 * 2  # gradient type x copy type (none, fp16, bf16) x decision record x device scalars


def test_uniform_values_come_through_scalar_loads(kernels):
    """By-value variants: nothing wave-uniform is fetched with a vector load (those show up as
    global loads with a scalar base register), and the decision record is read with s_load."""
    for name, _, _, has_ctl, has_hyper, body in _tile_variants(kernels):
        if has_hyper:
            continue
        uniform_vector_loads = re.findall(r"global_load_\w+\s+v[\[\d:\]]+, v\d+, s\[", body)
        assert not uniform_vector_loads, (name, uniform_vector_loads)
        scalar_record_loads = re.findall(r"s_load_dword\s+s\d+, s\[\d+:\d+\], 0x[04]\b", body)
        assert (len(scalar_record_loads) >= 2) == has_ctl, (name, scalar_record_loads)


def test_tile_traffic_is_streaming(kernels):
    """Per-lane loads are all non-temporal, stores all streaming buffer stores; their number is that of
    the arrays (plus the three copy-through pairs of a skipped out-of-place step)."""
    for name, g, h, has_ctl, _, body in _tile_variants(kernels):
        lane_loads = re.findall(r"global_load_dwordx[24]\s+v\[\d+:\d+\], v\[\d+:\d+\], off(.*)", body)
        assert len(lane_loads) == 4 + (3 if has_ctl else 0) and all(" nt" in tail for tail in lane_loads), (name, lane_loads)
        stores = re.findall(r"buffer_store_dwordx([24]) (.*)", body)
        assert all(tail.rstrip().endswith("offen nt sc1") for _, tail in stores), (name, stores)
        widths = [w for w, _ in stores]
        assert widths.count("4") == 3 + (3 if has_ctl else 0) and widths.count("2") == (0 if h == "n1" else 1), (name, widths)
        assert "global_store" not in body and "scratch_" not in body, name


def test_no_kernel_spills(kernels):
    for name, body in kernels.items():
        assert "scratch_" not in body, name


def test_statistics_pass_has_a_streaming_and_a_caching_load_path(kernels):
    """The statistics pass reads the part of the gradients that the update will want again with
    caching buffer loads and everything else with non-temporal loads: both instructions must have
    survived (a compiler that merges the two branches drops the streaming hint)."""
    seen = 0
    for name, body in kernels.items():
        if "grad_stats_kernel" not in name:
            continue
        seen += 1
        assert re.search(r"global_load_dwordx4 .* nt", body), name
        assert re.search(r"buffer_load_dwordx4 ", body), name
    assert seen == 3  # one per gradient type


def test_many_segment_kernel_keeps_its_table_in_scalar_registers(kernels):
    """The segment search is scalar compares and selects over the kernel arguments; the segment's
    record comes through scalar loads at a computed offset (no private copy of the table, which
    would show up as scratch or as vector loads of the arguments)."""
    seen = 0
    for name, body in kernels.items():
        if "adam_multi_kernel" not in name:
            continue
        seen += 1
        assert len(re.findall(r"s_cselect_b32", body)) >= 15, name
        assert re.search(r"s_load_dwordx\d+ s\[\d+:\d+\], s\[\d+:\d+\], s\d+", body), name  # register offset: the computed record address
    assert seen == 3 * 3 * 2 * 2


def test_relaxed_alignment_kernel_uses_full_width_accesses(kernels):
    """Arrays whose alignments disagree are still moved 16 (8) bytes per lane and instruction, and the
    loads of a tile are issued back to back: the three variants differ in which array is read with the
    default cache policy (a buffer load) instead of streaming, and must not make a load wait for the
    one before it (a run-time choice of the load instruction per array once did: every load was
    followed by s_waitcnt vmcnt(0))."""
    seen = 0
    for name, body in kernels.items():
        if "adam_tile_relaxed_kernel" not in name:
            continue
        seen += 1
        has_ctl, cached = re.search(r"ELb([01])ELi(\d)EEEv", name).groups()  # the last two template arguments
        has_ctl, cached = has_ctl == "1", int(cached)
        fp32_g = "kernelILi0E" in name
        streaming = len(re.findall(r"global_load_dwordx4 .* nt", body))
        buffered = len(re.findall(r"buffer_load_dwordx[24] ", body))
        # a skipped out-of-place step copies the three state arrays through: three more streaming loads
        assert streaming == 3 + (1 if fp32_g else 0) - (1 if cached == 1 else 0) - (1 if cached == 2 and fp32_g else 0) \
            + (3 if has_ctl else 0), name
        assert buffered == (1 if cached else 0), name
        assert len(re.findall(r"global_store_dwordx4 .* nt", body)) >= 3, name
        assert not re.search(r"global_(load|store)_(ubyte|short|ushort)", body), name
        assert "flat_load" not in body and "flat_store" not in body, name
        # the four loads of a tile (gradient, p, m, v) follow one another with no wait for a load between them
        loads = [m.start() for m in re.finditer(r"(global|buffer)_load_dwordx[24] ", body)]
        assert any("s_waitcnt vmcnt" not in body[loads[k]:loads[k + 3]] for k in range(len(loads) - 3)), name
    assert seen == 3 * 3 * 2 * 3
