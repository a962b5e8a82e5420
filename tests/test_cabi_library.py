"""The C-ABI library loads without a GPU, exports every symbol the header declares, and its pure
or argument-checking entry points behave (no compute call is made here)."""

import ctypes
import shutil
import subprocess

import pytest

import cabi
from oracle import nanoep_oracle as oracle


def test_every_declared_symbol_is_exported():
    declared = cabi.declared_symbols()
    assert {"nanoep_layout", "nanoep_dispatch", "nanoep_combine", "nanoep_wait_counts", "nanoep_window_layout",
            "nanoep_layout_workspace_bytes", "nanoep_copy_bytes", "nanoep_abi_version",
            "nanoep_slot_order_entries", "nanoep_layout_block_tokens", "nanoep_layout_static", "nanoep_rebuild_order",
            "nanoep_rebuild_workspace_bytes", "nanoep_rebuild_window_tokens", "nanoep_stream_probe", "nanoep_set_tuning",
            "nanoep_get_tuning", "nanoep_reset_tuning", "nanoep_device_topology"} <= set(declared)
    library = cabi.lib()
    for name in declared:
        assert hasattr(library, name), f"{name} is declared in include/nanoep_hip.h but not exported"


def test_version_and_status_strings():
    library = cabi.lib()
    assert library.nanoep_abi_version() == 4
    texts = [library.nanoep_status_string(code).decode() for code in range(0, 8)]
    assert texts[0] == "ok" and len(set(texts[:7])) == 7 and texts[7] == "unknown status"
    assert "static scratch" in texts[6] and "4 MiB" in texts[6]
    assert library.nanoep_last_hip_error().decode() == ""


@pytest.mark.parametrize("args", [(2, 8, 256, 2, 4, False), (1, 16, 256, 2, 2, False), (8, 4096, 7168, 8, 256, True),
                                  (4, 5, 512, 3, 12, True), (1, 32768, 7168, 8, 32, False)])
def test_window_layout_matches_the_oracle(args):
    assert cabi.window_layout(*args) == oracle.window_layout(*args)


def test_window_layout_known_answer_and_errors():
    assert cabi.window_layout(2, 8, 256, 2, 4) == [0, 96, 160, 160, 9888]
    out = (ctypes.c_int64 * 5)()
    library = cabi.lib()
    for bad in ((0, 8, 256, 2, 4), (33, 8, 256, 2, 64), (2, 0, 256, 2, 4), (2, 8, 0, 2, 4), (2, 8, 256, 33, 4), (2, 8, 256, 2, 5)):
        assert library.nanoep_window_layout(*bad, 0, out) == 1


def test_workspace_size_grows_with_the_problem():
    library = cabi.lib()
    small = library.nanoep_layout_workspace_bytes(16, 2, 2)
    large = library.nanoep_layout_workspace_bytes(4096, 8, 256)
    assert 0 < small < large
    assert large >= 4096 * 8 * 4 + 4096 * 4 + (4096 // 256) * 257 * 4
    assert library.nanoep_layout_workspace_bytes(-1, 8, 256) == 0
    assert library.nanoep_layout_workspace_bytes(16, 0, 2) == 0


def test_argument_checks_come_before_any_device_work():
    library = cabi.lib()
    null = None
    # hidden not a multiple of 8, top-k out of range, negative counts, unaligned pointers
    assert library.nanoep_dispatch(null, null, null, null, null, null, 0, null, null, 0, 0, 0, 7, 2, 4, 1, 0, 0, null, null, null, 0, null) == 1
    assert library.nanoep_dispatch(null, null, null, null, null, null, 0, null, null, 0, 0, 0, 256, 33, 4, 1, 0, 0, null, null, null, 0, null) == 1
    assert library.nanoep_dispatch(null, null, null, null, null, null, 0, null, null, 5, 0, 4, 256, 2, 4, 1, 0, 0, null, null, null, 0, null) == 1
    assert library.nanoep_dispatch(8, null, null, null, null, null, 0, null, null, 0, 0, 0, 256, 2, 4, 1, 0, 0, null, null, null, 0, null) == 1
    assert library.nanoep_combine(null, null, null, null, null, null, 0, 0, 0, 250, 2, 1, 0, null, null, 0, null) == 1
    assert library.nanoep_combine(null, null, null, null, null, null, 3, 0, 2, 256, 2, 1, 0, null, null, 0, null) == 1
    assert library.nanoep_copy_bytes(null, null, 24, null) == 1
    assert library.nanoep_layout(null, -1, 2, 4, 1, 0, 0, null, null, null, null, null, null, null, null, null, null, 0, null, null) == 1
    assert library.nanoep_layout(null, 4, 2, 4, 0, 0, 0, null, null, null, null, null, null, null, null, null, null, 0, null, null) == 1
    # a slot-order list only exists for the expanded layout
    assert library.nanoep_layout(null, 4, 2, 4, 1, 0, 0, null, 8, 8, null, 8, null, 8, null, 8, 8, 0, 8, null) == 1
    assert library.nanoep_slot_order_entries(4096, 8, 256) == 4096 * 8 + 1 and library.nanoep_layout_block_tokens(4096, 256, 0) == 256
    assert library.nanoep_slot_order_entries(100, 3, 8) == 256 * 3 + 1 and library.nanoep_slot_order_entries(0, 3, 8) == 0
    assert library.nanoep_layout_block_tokens(4096, 6000, 0) == 0 and library.nanoep_layout_block_tokens(4096, 0, 0) == 0
    # most local experts: four int32 per expert (and one more row) in 60 KiB of LDS
    assert library.nanoep_layout_block_tokens(4096, 3839, 0) == 256 and library.nanoep_layout_block_tokens(4096, 3840, 0) == 0
    sizes = (1, 256, 257, 512, 1024, 1536, 1792, 1793, 2048, 4095, 4096, 100000)
    for hidden in (0, 7168):
        assert [library.nanoep_layout_block_tokens(t, 256, hidden) for t in sizes] == [256, 256, 64, 64, 128, 128, 128, 256, 256, 256, 256, 256]
    # rows of up to 4096 elements: windows of 512 tokens (two layout blocks) once there are eight of them
    assert [library.nanoep_layout_block_tokens(t, 256, 2048) for t in sizes] == [256, 256, 64, 64, 128, 128, 128, 256, 256, 512, 512, 512]
    # a window's rows fit an XCD's 4 MiB L2
    assert [library.nanoep_layout_block_tokens(100000, 256, h) for h in (8, 1024, 1032, 3840, 3848, 7680, 7688, 15360, 15368, 1 << 20)] == [1024, 1024, 512, 512, 256, 256, 128, 128, 64, 64]
    # windows of 1024 tokens (rows of up to 1024 elements) once there are sixteen of them
    assert [library.nanoep_layout_block_tokens(t, 256, 1024) for t in (4096, 15360, 15361, 16384)] == [512, 512, 1024, 1024]
    assert library.nanoep_layout_block_tokens(100000, 1400, 2048) == 512  # four layout blocks of 128 tokens (1401 LDS rows)
    assert library.nanoep_layout_block_tokens(100000, 1400, 512) == 1024  # eight of them
    assert library.nanoep_layout_block_tokens(300000, 256, 2048) == 256  # separate scan launch: the window is the layout block
    assert library.nanoep_layout_block_tokens(4096, 256, -1) == 0
    out = (ctypes.c_int64 * 4)()
    assert library.nanoep_wait_counts(null, null, 0.0, out) == 1


def test_tuning_switches_are_set_through_the_abi_and_read_from_the_environment_once(monkeypatch):
    """The switches are parsed from NANOEP_<NAME> once; afterwards only nanoep_set_tuning changes
    them (an environment variable set later is not seen until nanoep_reset_tuning reads it)."""
    library = cabi.lib()
    assert cabi.get_tuning("WINDOW_TOKENS") == 0 and cabi.get_tuning("DISPATCH_ORDER") == -1 and cabi.get_tuning("XCDS") == 0
    assert cabi.get_tuning("DISPATCH_PREFETCH") == -1 and cabi.get_tuning("COMBINE_STORES") == -1 and cabi.get_tuning("DISPATCH_SPAN") == 0
    assert cabi.get_tuning("DISPATCH_PACK") == 0 and cabi.get_tuning("COMBINE_UNITS") == 0
    value = ctypes.c_int(0)
    assert library.nanoep_get_tuning(b"NO_SUCH_SWITCH", ctypes.byref(value)) == 1
    assert library.nanoep_set_tuning(b"NO_SUCH_SWITCH", 3) == 1 and library.nanoep_set_tuning(None, 3) == 1
    try:
        assert library.nanoep_set_tuning(b"WINDOW_TOKENS", 128) == 0
        assert cabi.get_tuning("WINDOW_TOKENS") == 128
        assert library.nanoep_layout_block_tokens(4096, 256, 7168) == 128  # the forced window shows in the plan
        monkeypatch.setenv("NANOEP_WINDOW_TOKENS", "192")
        assert library.nanoep_layout_block_tokens(4096, 256, 7168) == 128  # the environment is not read again by a call
        with cabi.forced_tuning({"WINDOW_TOKENS": 64, "DISPATCH_SPAN": None}):
            assert cabi.get_tuning("WINDOW_TOKENS") == 64
        assert cabi.get_tuning("WINDOW_TOKENS") == 128
        library.nanoep_reset_tuning()
        assert cabi.get_tuning("WINDOW_TOKENS") == 192
    finally:
        monkeypatch.delenv("NANOEP_WINDOW_TOKENS", raising=False)
        library.nanoep_reset_tuning()
    assert cabi.get_tuning("WINDOW_TOKENS") == 0 and library.nanoep_layout_block_tokens(4096, 256, 7168) == 256


def test_topology_defaults_and_overrides_size_the_windows():
    """Without a device the plans assume the MI355X's 256 CUs, 8 XCDs and 4 MiB of L2 per XCD; the
    XCDS and L2_BYTES switches stand in for other parts: the window follows the L2, the number of
    windows a batch is cut into follows the XCD count."""
    library = cabi.lib()
    assert cabi.device_topology() == (256, 8, 4 << 20)
    try:
        library.nanoep_set_tuning(b"L2_BYTES", 8 << 20)
        assert cabi.device_topology() == (256, 8, 8 << 20)
        assert [library.nanoep_layout_block_tokens(100000, 256, h) for h in (2048, 4096, 8192, 16384)] == [1024, 512, 256, 128]
        library.nanoep_set_tuning(b"L2_BYTES", 2 << 20)
        assert [library.nanoep_layout_block_tokens(100000, 256, h) for h in (3840, 7680, 16384)] == [256, 128, 64]
        library.nanoep_set_tuning(b"L2_BYTES", 0)
        library.nanoep_set_tuning(b"XCDS", 4)
        assert cabi.device_topology() == (256, 4, 4 << 20)
        # 1024 tokens of 7168 elements: eight windows of 128 tokens for 8 XCDs, four of 256 for 4
        assert library.nanoep_layout_block_tokens(1024, 256, 7168) == 256
        library.nanoep_set_tuning(b"XCDS", 0)
        assert library.nanoep_layout_block_tokens(1024, 256, 7168) == 128
    finally:
        library.nanoep_reset_tuning()


def test_rebuild_and_stream_probe_argument_checks():
    library = cabi.lib()
    null = None
    assert library.nanoep_rebuild_workspace_bytes(4096, 8) >= (4096 // 32) * 4 and library.nanoep_rebuild_workspace_bytes(-1, 8) == 0
    assert library.nanoep_rebuild_workspace_bytes(16, 0) == 0 and library.nanoep_rebuild_workspace_bytes(16, 33) == 0
    # the layout's window, halved until a window's T * K entries fit the sort (4096)
    assert library.nanoep_rebuild_window_tokens(4096, 8, 7168) == 256 and library.nanoep_rebuild_window_tokens(8192, 8, 2048) == 512
    assert library.nanoep_rebuild_window_tokens(32768, 8, 512) == 512 and library.nanoep_rebuild_window_tokens(4096, 32, 7168) == 128
    assert library.nanoep_rebuild_window_tokens(4096, 0, 7168) == 0
    # no tokens, missing pointers, a tag with low bits, a negative tag, too many (token, k) pairs
    assert library.nanoep_rebuild_order(8, 8, 0, 0, 0, 2, 4, 256, 8, 8, 8, 1024, null, 0, null) == 1
    assert library.nanoep_rebuild_order(8, null, 1, 4, 4, 2, 4, 256, 8, 8, 8, 1024, null, 0, null) == 1
    assert library.nanoep_rebuild_order(8, 8, 1, 4, 4, 2, 4, 256, 8, 8, 8, 1024, null, 5, null) == 1
    assert library.nanoep_rebuild_order(8, 8, 1, 4, 4, 2, 4, 256, 8, 8, 8, 1024, null, -(1 << 32), null) == 1
    assert library.nanoep_rebuild_order(8, 8, 1, 4, 1 << 30, 8, 4, 256, 8, 8, 8, 1 << 30, null, 0, null) == 1
    assert library.nanoep_rebuild_order(8, 8, 5, 4, 4, 2, 4, 256, 8, 8, 8, 1024, null, 0, null) == 1  # more rows than tokens
    assert library.nanoep_rebuild_order(8, 8, 1, 4, 4, 2, 4, 256, 8, 8, 8, 16, null, 0, null) == 3  # workspace too small
    library.nanoep_stream_probe.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    for bad in ((4, 16, 16, 64, 256, 1, 1, 0), (2, 16, 16, 64, 250, 1, 1, 0), (2, 16, 16, 64, 16384, 1, 1, 0), (2, 16, 16, 64, 256, 3, 1, 0),
                (2, 16, 16, 64, 256, 2, 64, 0), (3, 16, 16, 60, 256, 2, 64, 0), (2, 16, 16, 64, 256, 2, 1, 17), (2, null, 16, 64, 256, 2, 1, 0),
                (1, null, null, 64, 256, 1, 1, 0), (0, 16, 24, 64, 256, 1, 1, 0)):
        assert library.nanoep_stream_probe(*bad, null) == 1, bad


def test_wait_counts_reads_a_mailbox_the_host_wrote():
    """nanoep_wait_counts against a mailbox in plain host memory, no GPU involved: published counts
    come back whole, a routing status word turns into NANOEP_ERR_ROUTING with the words still
    delivered, and a word that never arrives ends in NANOEP_ERR_TIMEOUT once the caller's patience
    (none here) is used up, before the stream is ever looked at."""
    library = cabi.lib()
    mailbox = (ctypes.c_int64 * 4)(17, 40, 33, 0)
    out = (ctypes.c_int64 * 4)()
    assert library.nanoep_wait_counts(mailbox, None, 0.0, out) == 0 and list(out) == [17, 40, 33, 0]
    # N == 0 is a count like any other
    mailbox[:] = [0, 0, 0, 0]
    assert library.nanoep_wait_counts(mailbox, None, 0.0, out) == 0 and list(out) == [0, 0, 0, 0]
    for status_word in (1, 2, 3):
        mailbox[:] = [5, 9, 8, status_word]
        assert library.nanoep_wait_counts(mailbox, None, 0.0, out) == 5 and list(out) == [5, 9, 8, status_word]
    # word 0 still -1 (what nanoep_layout leaves there until the device has stored the rest)
    mailbox[:] = [-1, 40, 33, 0]
    out[:] = [7, 7, 7, 7]
    assert library.nanoep_wait_counts(mailbox, None, 0.0, out) == 4
    assert list(out) == [7, 7, 7, 7]  # nothing is delivered from an unpublished mailbox
    assert b"timed out" in library.nanoep_status_string(4)
    # ... and a late store is only seen by a later wait
    mailbox[0] = 3
    assert library.nanoep_wait_counts(mailbox, None, 0.0, out) == 0 and list(out) == [3, 40, 33, 0]


def test_static_layout_checks_arguments_and_its_size_limit_before_any_device_work():
    library = cabi.lib()
    null = None
    assert library.nanoep_layout_static(null, -1, 2, 4, 1, 0, 0, null, null, null, null, null, null, null, null, null, null, null) == 1
    assert library.nanoep_layout_static(null, 4, 2, 4, 1, 0, 0, null, 8, 8, null, 8, null, 8, null, 8, 8, null) == 1
    # 4 MiB of static scratch: the headline batch needs 0.2 MiB, 32768 tokens 1.7 MiB, 131072 tokens x top-8 more than 4
    assert library.nanoep_layout_workspace_bytes(4096, 8, 256) < library.nanoep_layout_workspace_bytes(32768, 8, 256) < (4 << 20)
    assert library.nanoep_layout_workspace_bytes(131072, 8, 256) > (4 << 20)
    assert library.nanoep_layout_static(8, 131072, 8, 256, 1, 1, 0, 8, 8, 8, 8, 8, 8, 8, 8, 8, 8, null) == 6


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")
def test_plain_c_client_compiles_links_and_runs(tmp_path):
    """The header is C99 and the library links from C without HIP or torch on the include path."""
    binary = tmp_path / "cabi_c_client"
    source = cabi.ROOT / "tests" / "cabi_c_client.c"
    library_dir = cabi.LIBRARY.parent
    subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{cabi.HEADER.parent}", str(source), "-o", str(binary),
         f"-L{library_dir}", "-lnanoep_hip", f"-Wl,-rpath,{library_dir}"],
        check=True, capture_output=True, text=True,
    )
    out = subprocess.run([str(binary)], check=True, capture_output=True, text=True, timeout=60).stdout.splitlines()
    assert out[0] == "abi 4 status 0 window 0 96 160 160 9888"
    assert out[1].startswith("invalid 1 '") and "invalid" in out[1].lower()
    assert out[2] == "sizes 32769 256 1"
