"""ctypes binding of include/nanoep_hip.h for the tests: torch supplies device memory and streams,
every compute call goes through the C ABI of nanoep_amd/libnanoep_hip.so."""

from __future__ import annotations

import contextlib
import ctypes
import re
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parent.parent
LIBRARY = ROOT / "nanoep_amd" / "libnanoep_hip.so"
HEADER = ROOT / "include" / "nanoep_hip.h"

HOST_COUNT_WORDS = 4


def declared_symbols() -> list[str]:
    """Function names declared in the public header."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(nanoep_[a-z0-9_]+)\s*\(", text)))


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIBRARY.exists():
            raise RuntimeError(f"{LIBRARY} is missing: run `python -m nanoep_amd.build` first")
        handle = ctypes.CDLL(str(LIBRARY))
        p, i, i64, sz, dbl = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_double
        handle.nanoep_abi_version.restype = i
        handle.nanoep_status_string.restype = ctypes.c_char_p
        handle.nanoep_status_string.argtypes = [i]
        handle.nanoep_last_hip_error.restype = ctypes.c_char_p
        handle.nanoep_device_cu_count.argtypes = [i, ctypes.POINTER(i)]
        handle.nanoep_window_layout.argtypes = [i, i64, i, i, i64, i, ctypes.POINTER(i64)]
        handle.nanoep_layout_workspace_bytes.restype = sz
        handle.nanoep_layout_workspace_bytes.argtypes = [i64, i, i64]
        handle.nanoep_layout_block_tokens.restype = i
        handle.nanoep_layout_block_tokens.argtypes = [i64, i64, i]
        handle.nanoep_slot_order_entries.restype = i64
        handle.nanoep_slot_order_entries.argtypes = [i64, i, i64]
        handle.nanoep_layout.argtypes = [p, i64, i, i64, i64, i, i, p, p, p, p, p, p, p, p, p, p, sz, p, p]
        handle.nanoep_layout_static.argtypes = [p, i64, i, i64, i64, i, i, p, p, p, p, p, p, p, p, p, p, p]
        handle.nanoep_wait_counts.argtypes = [p, p, dbl, ctypes.POINTER(i64)]
        handle.nanoep_dispatch.argtypes = [p, p, p, p, p, p, i64, p, p, i64, i64, i64, i, i, i64, i64, i, i, p, p, p, i, p]
        handle.nanoep_combine.argtypes = [p, p, p, p, p, p, i64, i64, i64, i, i, i, i, p, p, i, p]
        handle.nanoep_copy_bytes.argtypes = [p, p, sz, p]
        handle.nanoep_rebuild_window_tokens.argtypes = [i64, i, i]
        handle.nanoep_rebuild_workspace_bytes.restype = sz
        handle.nanoep_rebuild_workspace_bytes.argtypes = [i64, i]
        handle.nanoep_rebuild_order.argtypes = [p, p, i64, i64, i64, i, i64, i, p, p, p, sz, p, i64, p]
        handle.nanoep_set_tuning.argtypes = [ctypes.c_char_p, i]
        handle.nanoep_get_tuning.argtypes = [ctypes.c_char_p, ctypes.POINTER(i)]
        handle.nanoep_reset_tuning.restype = None
        handle.nanoep_device_topology.argtypes = [ctypes.POINTER(i), ctypes.POINTER(i), ctypes.POINTER(i64)]
        _lib = handle
    return _lib


class NanoEPError(RuntimeError):
    def __init__(self, status: int):
        self.status = status
        detail = lib().nanoep_last_hip_error().decode()
        super().__init__(f"nanoep status {status}: {lib().nanoep_status_string(status).decode()} {detail}".strip())


def check(status: int) -> None:
    if status != 0:
        raise NanoEPError(status)


def ptr(tensor: torch.Tensor | None):
    return None if tensor is None or tensor.numel() == 0 and tensor.data_ptr() == 0 else tensor.data_ptr()


def stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


def get_tuning(name: str) -> int:
    value = ctypes.c_int(0)
    check(lib().nanoep_get_tuning(name.encode(), ctypes.byref(value)))
    return value.value


@contextlib.contextmanager
def forced_tuning(switches: dict):
    """Sets the given tuning switches (None: leave alone) through the C ABI and puts the previous values back."""
    previous = {name: get_tuning(name) for name, value in switches.items() if value is not None}
    try:
        for name in previous:
            check(lib().nanoep_set_tuning(name.encode(), int(switches[name])))
        yield
    finally:
        for name, value in previous.items():
            check(lib().nanoep_set_tuning(name.encode(), value))


def device_topology() -> tuple[int, int, int]:
    cus, xcds, l2 = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int64(0)
    check(lib().nanoep_device_topology(ctypes.byref(cus), ctypes.byref(xcds), ctypes.byref(l2)))
    return cus.value, xcds.value, l2.value


def window_layout(ranks, tokens, hidden, topk, experts, multi=False) -> list[int]:
    out = (ctypes.c_int64 * 5)()
    check(lib().nanoep_window_layout(ranks, tokens, hidden, topk, experts, int(multi), out))
    return list(out)


def layout(topk_idx: torch.Tensor, num_local_experts: int, alignment: int, expand: bool, *, raise_on_routing=True, hidden=0,
           static_scratch=False):
    """Runs the layout kernels and returns (metadata list of 7, or 9 when expanded, (N, C, A, status)).
    hidden is the row width the handle will be used with (0: not known); it sizes the token blocks.
    static_scratch takes nanoep_layout_static (the library's own device array) instead of nanoep_layout."""
    device = topk_idx.device
    tokens, topk = topk_idx.shape
    i64 = dict(dtype=torch.int64, device=device)
    recv_metadata = torch.empty((tokens, topk + 2), dtype=torch.int32, device=device)
    expert_counts = torch.empty(num_local_experts, **i64)
    expert_offsets = torch.empty(num_local_experts + 1, **i64)
    dst_slots = torch.empty((tokens, 1), **i64)
    send_counts = torch.empty(1, **i64)
    snapshot = torch.empty_like(topk_idx)
    prefix = torch.empty(1, **i64)
    token_slots = torch.empty((tokens, topk), dtype=torch.int32, device=device) if expand else None
    slot_order = None
    if expand:
        entries = lib().nanoep_slot_order_entries(tokens, topk, num_local_experts)
        slot_order = torch.full((entries,), -7, dtype=torch.int64, device=device)
    mailbox = torch.empty(HOST_COUNT_WORDS, dtype=torch.int64, pin_memory=True)
    if static_scratch:
        check(
            lib().nanoep_layout_static(
                ptr(topk_idx), tokens, topk, num_local_experts, alignment, int(expand), hidden, ptr(recv_metadata),
                ptr(expert_counts), ptr(expert_offsets), ptr(dst_slots), ptr(send_counts), ptr(snapshot), ptr(prefix),
                ptr(token_slots), ptr(slot_order), mailbox.data_ptr(), stream_handle(),
            )
        )
    else:
        ws_bytes = lib().nanoep_layout_workspace_bytes(tokens, topk, num_local_experts)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
        check(
            lib().nanoep_layout(
                ptr(topk_idx), tokens, topk, num_local_experts, alignment, int(expand), hidden, ptr(recv_metadata),
                ptr(expert_counts), ptr(expert_offsets), ptr(dst_slots), ptr(send_counts), ptr(snapshot), ptr(prefix),
                ptr(token_slots), ptr(slot_order), ptr(workspace), ws_bytes, mailbox.data_ptr(), stream_handle(),
            )
        )
    out = (ctypes.c_int64 * HOST_COUNT_WORDS)()
    status = lib().nanoep_wait_counts(mailbox.data_ptr(), stream_handle(), 30.0, out)
    if status != 0 and (raise_on_routing or status != 5):
        raise NanoEPError(status)
    counts = tuple(out)
    torch.cuda.current_stream().synchronize()  # workspace and mailbox may be released
    metadata = [recv_metadata[: counts[0]], expert_counts, expert_offsets, dst_slots, send_counts, snapshot, prefix]
    if token_slots is not None:
        metadata.append(token_slots)  # private eighth entry: the one-lookup slot table
        metadata.append(slot_order)  # private ninth entry: assignments in block-wise slot order
    return metadata, counts


def rebuild_order(metadata, counts, num_local_experts, hidden, *, host_tag=None):
    """The private tensors of an expanded handle rebuilt from its recv_metadata and dst_slots alone
    (nanoep_rebuild_order): returns (token_slots, slot_order, published word or None)."""
    recv_metadata, dst_slots = metadata[0], metadata[3]
    device = dst_slots.device
    tokens = dst_slots.shape[0]
    topk = recv_metadata.shape[1] - 2
    table = torch.full((tokens, topk), -9, dtype=torch.int32, device=device)
    order = torch.full((lib().nanoep_slot_order_entries(tokens, topk, num_local_experts),), -7, dtype=torch.int64, device=device)
    nbytes = lib().nanoep_rebuild_workspace_bytes(tokens, topk)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    word = torch.full((1,), -5, dtype=torch.int64).pin_memory() if host_tag is not None else None
    check(lib().nanoep_rebuild_order(ptr(recv_metadata), ptr(dst_slots), counts[0], counts[1], tokens, topk, num_local_experts, hidden,
                                     ptr(table), ptr(order), ptr(workspace), nbytes, None if word is None else word.data_ptr(),
                                     0 if host_tag is None else host_tag, stream_handle()))
    torch.cuda.current_stream().synchronize()
    return table, order, None if word is None else int(word[0])


def token_slots_of(metadata, use_table=True):
    return metadata[7] if use_table and len(metadata) > 7 else None


def slot_order_of(metadata, use_order=True):
    return metadata[8] if use_order and len(metadata) > 8 else None


def dispatch(x, weights, metadata, counts, num_local_experts, alignment, expand, zero_padding, *, num_cus=0, poison=None,
             use_table=True, use_order=True, order_count="exact", walk="forced", span=None, rows=None, prefetch=None, pack=None):
    """Returns (recv_x, recv_topk_idx | None, recv_weights | None) through nanoep_dispatch.

    walk="forced" sets the library's switch for the slot-order walk explicitly, walk="auto" leaves
    the switch alone (the library then walks the list whenever it is given one).  span=1|2|4
    forces the number of chunks a wavefront of that walk moves (the library picks it by source size).
    rows=n asks for n list entries a workgroup of that walk (honoured for rows of up to four pieces while
    the workgroup stays within 16 wavefronts).  prefetch=0|1 forbids or asks for that walk's window-wise
    source prefetch.  pack=1 keeps one list entry a wavefront for rows of at most 512 bytes (the library
    packs four or eight).
    """
    recv_metadata, expert_counts, expert_offsets, dst_slots = metadata[0], metadata[1], metadata[2], metadata[3]
    received, capacity = counts[0], counts[1]
    tokens, hidden = x.shape
    topk = recv_metadata.shape[1] - 2
    rows = capacity if expand else received
    device = x.device

    def new(shape, dtype):
        out = torch.empty(shape, dtype=dtype, device=device)
        if poison is not None and out.numel():
            out.view(torch.uint8).fill_(poison)
        return out

    recv_x = new((rows, hidden), torch.bfloat16)
    recv_idx = None if expand else new((rows, topk), torch.int64)
    recv_w = None if weights is None else new((rows,) if expand else (rows, topk), torch.float32)
    order = slot_order_of(metadata, use_order)
    # exact count A, or -1: the kernel reads A from the word behind the list
    # ... or -g: the same, with the launch sized for about g entries (order_count=("device", g))
    if order is None:
        order_entries = 0
    elif order_count == "exact":
        order_entries = counts[2]
    else:
        order_entries = -1 if order_count == "device" else -int(order_count[1])
    switches = {"DISPATCH_ORDER": 1 if walk == "forced" else None, "DISPATCH_SPAN": span,
                "ROWS_PER_BLOCK": rows, "DISPATCH_PACK": pack,
                "DISPATCH_PREFETCH": None if prefetch is None else int(prefetch)}
    with forced_tuning(switches):
        status = lib().nanoep_dispatch(
            ptr(x), ptr(weights), ptr(recv_metadata), ptr(dst_slots), ptr(token_slots_of(metadata, use_table)),
            ptr(order), order_entries, ptr(expert_counts), ptr(expert_offsets), received, capacity,
            tokens, hidden, topk, num_local_experts, alignment, int(expand), int(zero_padding), ptr(recv_x),
            ptr(recv_idx), ptr(recv_w), num_cus, stream_handle(),
        )
    check(status)
    return recv_x, recv_idx, recv_w


def combine(y, weights, bias, metadata, counts, expand, *, multiple_reduction=False, num_cus=0, poison=None, use_table=True,
            stores=None, units=None):
    """Returns (out_x [T,H], out_weights [T,K] | None) through nanoep_combine.  stores=0|1 asks for
    nontemporal / agent-scope stores of the output rows (the library picks by output size);
    units=1..16 for that many tokens a wavefront where the library has a choice (five or more
    rows a token with the slot table; it picks by batch size)."""
    recv_metadata, dst_slots = metadata[0], metadata[3]
    tokens = dst_slots.shape[0]
    topk = recv_metadata.shape[1] - 2
    hidden = y.shape[1]
    device = y.device
    out_x = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=device)
    out_w = None if weights is None else torch.empty((tokens, topk), dtype=torch.float32, device=device)
    if poison is not None:
        for tensor in (out_x, out_w):
            if tensor is not None and tensor.numel():
                tensor.view(torch.uint8).fill_(poison)
    with forced_tuning({"COMBINE_STORES": stores, "COMBINE_UNITS": units}):
        check(
            lib().nanoep_combine(
                ptr(y), ptr(weights), ptr(bias), ptr(recv_metadata), ptr(dst_slots), ptr(token_slots_of(metadata, use_table)), counts[0],
                y.shape[0], tokens,
                hidden, topk, int(expand), int(multiple_reduction), ptr(out_x), ptr(out_w), num_cus, stream_handle(),
            )
        )
    return out_x, out_w
