"""Thin torch-facing wrappers over the device C-ABI (include/df11.h).

torch is used for device memory and streams only; the work happens in
libdf11_hip.so.  There is no CPU path: these functions raise if the tensors are
not on a GPU or the library cannot be loaded.
"""
import torch

from . import _native


# The handle of a device's current stream without building a torch.cuda.Stream object
# around it (the hook asks for it before every launch).
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device):
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(**tensors):
    for name, t in tensors.items():
        if not t.is_cuda:
            raise _native.DF11Error(f"{name} must live on the GPU (got {t.device}); there is no CPU decode path")
        if not t.is_contiguous():
            raise _native.DF11Error(f"{name} must be contiguous")


def workspace_bytes(n_bytes):
    return int(_native.hip_lib().df11_workspace_bytes(int(n_bytes)))


def _check_stream_tensors(luts, encoded_exponent, output_positions, gaps):
    if luts.dtype != torch.uint8 or luts.dim() != 2 or luts.shape[1] != 256 or luts.shape[0] < 2:
        raise _native.DF11Error(f"luts must be uint8 [n_luts >= 2, 256], got {luts.dtype} {tuple(luts.shape)}")
    n_blocks = -(-encoded_exponent.numel() // 4096)
    if output_positions.numel() * output_positions.element_size() < 4 * n_blocks:
        raise _native.DF11Error("output_positions shorter than one entry per bitstream block")
    if gaps.numel() < 320 * n_blocks:
        raise _native.DF11Error("gaps shorter than 320 bytes per bitstream block")


def validate_stream(luts, encoded_exponent, sign_mantissa, output_positions, gaps, name="stream"):
    """Load-time check of one DF11 stream's layout (any device; reads the block
    positions on the host).  The reference decodes whatever it is given; a stream
    that fails here would make it read or write out of bounds.  Raises DF11Error."""
    def bad(why):
        raise _native.DF11Error(f"{name}: malformed DF11 stream: {why}")

    if luts.dtype != torch.uint8 or luts.dim() != 2 or luts.shape[1] != 256 or luts.shape[0] < 2:
        bad(f"luts must be uint8 [n_luts >= 2, 256], got {luts.dtype} {tuple(luts.shape)}")
    if luts.shape[0] - 1 > 17:
        bad(f"{luts.shape[0] - 1} decode tables, but a pointer entry can name 16 beside the root")
    for label, t in (("encoded_exponent", encoded_exponent), ("sign_mantissa", sign_mantissa), ("gaps", gaps)):
        if t.dtype != torch.uint8 or t.dim() != 1:
            bad(f"{label} must be a flat uint8 tensor")
    n_bytes, n_elements = encoded_exponent.numel(), sign_mantissa.numel()
    n_blocks = -(-n_bytes // 4096)
    if n_elements >= 1 << 32:
        bad("more than 2^32 - 1 elements in one stream")
    if n_elements > 8 * n_bytes:
        bad(f"{n_elements} elements cannot come from {n_bytes} bytes of bitstream")
    if gaps.numel() != 320 * n_blocks:
        bad(f"gaps has {gaps.numel()} bytes, expected {320 * n_blocks}")
    pos = output_positions.detach().cpu().contiguous().view(torch.uint8)
    if pos.numel() % 4:
        bad("output_positions is not a whole number of 32-bit words")
    pos = pos.view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    if pos.numel() not in (n_blocks, n_blocks + 1):
        bad(f"output_positions has {pos.numel()} entries for {n_blocks} bitstream blocks")
    if pos.numel():
        if int(pos[0]) != 0:
            bad("the first block does not start at element 0")
        if bool((pos[1:] < pos[:-1]).any()):
            bad("block positions decrease")
        if bool((pos[1:] - pos[:-1] > 4096 * 8).any()):
            bad("a block claims more elements than it has bits")
        if pos.numel() == n_blocks + 1 and int(pos[-1]) != n_elements:
            bad(f"last position {int(pos[-1])} differs from the number of elements {n_elements}")
        if int(pos[-1]) > n_elements:
            bad("a block starts past the last element")


def prepare(luts, encoded_exponent, output_positions, gaps, n_elements, workspace=None):
    """Build the decode workspace of one stream (load time; waits for the current stream).
    Returns (workspace uint8 tensor, max_elems_per_subblock)."""
    import ctypes
    _require_cuda(luts=luts, encoded_exponent=encoded_exponent, output_positions=output_positions, gaps=gaps)
    _check_stream_tensors(luts, encoded_exponent, output_positions, gaps)
    n_bytes = encoded_exponent.numel()
    need = workspace_bytes(n_bytes)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=luts.device)
    else:
        _require_cuda(workspace=workspace)
        if workspace.numel() * workspace.element_size() < need:
            raise _native.DF11Error("workspace buffer too small")
    max_sub = ctypes.c_int32(0)
    with torch.cuda.device(luts.device):
        rc = _native.hip_lib().df11_prepare(
            luts.data_ptr(), encoded_exponent.data_ptr(), output_positions.data_ptr(), gaps.data_ptr(),
            luts.shape[0], n_bytes, int(n_elements), workspace.data_ptr(), ctypes.byref(max_sub),
            _stream_ptr(luts.device))
    _native.check(rc, "df11_prepare")
    return workspace, int(max_sub.value)


PLANS = {"auto": -1, "wide": 0, "deep": 1, "deepest": 2, "portable": 3}


def decode(luts, encoded_exponent, sign_mantissa, output_positions, gaps, out, workspace,
           max_elems_per_subblock=0, plan=None):
    """Decode one DF11 stream into `out` (bfloat16, >= n_elements) on the current stream.
    `plan` (a key or value of PLANS) pins the kernel's launch plan for this call only (tests
    and measurements); by default the library chooses per stream."""
    _require_cuda(luts=luts, encoded_exponent=encoded_exponent, sign_mantissa=sign_mantissa,
                  output_positions=output_positions, gaps=gaps, out=out, workspace=workspace)
    _check_stream_tensors(luts, encoded_exponent, output_positions, gaps)
    n_elements = sign_mantissa.numel()
    n_bytes = encoded_exponent.numel()
    if out.dtype != torch.bfloat16 or out.numel() < n_elements:
        raise _native.DF11Error("out must be a bfloat16 tensor with at least n_elements elements")
    if workspace.numel() * workspace.element_size() < workspace_bytes(n_bytes):
        raise _native.DF11Error("workspace buffer too small")
    args = (luts.data_ptr(), encoded_exponent.data_ptr(), sign_mantissa.data_ptr(),
            output_positions.data_ptr(), gaps.data_ptr(), out.data_ptr(),
            luts.shape[0], n_bytes, n_elements, workspace.data_ptr(), int(max_elems_per_subblock))
    with torch.cuda.device(out.device):
        if plan is None:
            rc = _native.hip_lib().df11_decode(*args, _stream_ptr(out.device))
        else:
            rc = _native.hip_lib().df11_decode_with_plan(*args, _stream_ptr(out.device),
                                                         int(PLANS.get(plan, plan)))
    _native.check(rc, "df11_decode" if plan is None else "df11_decode_with_plan")
    return out


def bind(luts, encoded_exponent, sign_mantissa, output_positions, gaps, out, workspace,
         max_elems_per_subblock=0):
    """Checks the tensors of one stream once and returns the argument tuple that
    launch() passes to df11_decode.  The tuple holds raw addresses: it is valid for
    as long as these very tensors are alive and unmoved."""
    _require_cuda(luts=luts, encoded_exponent=encoded_exponent, sign_mantissa=sign_mantissa,
                  output_positions=output_positions, gaps=gaps, out=out, workspace=workspace)
    _check_stream_tensors(luts, encoded_exponent, output_positions, gaps)
    n_elements = sign_mantissa.numel()
    n_bytes = encoded_exponent.numel()
    if out.dtype != torch.bfloat16 or out.numel() < n_elements:
        raise _native.DF11Error("out must be a bfloat16 tensor with at least n_elements elements")
    if workspace.numel() * workspace.element_size() < workspace_bytes(n_bytes):
        raise _native.DF11Error("workspace buffer too small")
    return (luts.data_ptr(), encoded_exponent.data_ptr(), sign_mantissa.data_ptr(),
            output_positions.data_ptr(), gaps.data_ptr(), out.data_ptr(),
            luts.shape[0], n_bytes, n_elements, workspace.data_ptr(), int(max_elems_per_subblock))


def decode_rows(luts, encoded_exponent, sign_mantissa, output_positions, gaps, out, workspace,
                max_elems_per_subblock, row_ids, row_elements):
    """Decode only the rows `row_ids` (int64 device tensor) of the stream's output, taken as a
    matrix of row_elements elements per row, into their places in `out` (full size)."""
    bound = bind(luts, encoded_exponent, sign_mantissa, output_positions, gaps, out, workspace,
                 max_elems_per_subblock)
    if not launch_rows(bound, out.device, row_ids, row_elements):
        raise _native.DF11Error("df11_decode_rows is not available on this device; decode the whole stream")
    return out


def launch_rows(bound, device, row_ids, row_elements):
    """df11_decode_rows with arguments from bind(): decodes the rows of the output matrix
    (row_elements elements each) that the int64 device tensor `row_ids` names, into
    their places in the bound output buffer; the rest of the buffer is left as it is.
    Returns False, with nothing launched, if the library has no row decode for this
    device (it then runs every stream through its portable kernel): the caller decodes
    the whole stream instead."""
    if row_ids.dtype != torch.int64 or row_ids.device != device or not row_ids.is_contiguous():
        raise _native.DF11Error("row_ids must be a contiguous int64 tensor on the stream's device")
    lib = _native.hip_lib()
    if torch.cuda.current_device() == device.index:
        rc = lib.df11_decode_rows(*bound, _stream_ptr(device), row_ids.data_ptr(), row_ids.numel(), int(row_elements))
    else:
        with torch.cuda.device(device):
            rc = lib.df11_decode_rows(*bound, _stream_ptr(device), row_ids.data_ptr(), row_ids.numel(),
                                      int(row_elements))
    if rc == _native.ERR_UNSUPPORTED:
        return False
    if rc:
        _native.check(rc, "df11_decode_rows")
    return True


def launch(bound, device):
    """df11_decode with arguments from bind(), on the current stream of `device`."""
    lib = _native.hip_lib()
    if torch.cuda.current_device() == device.index:
        rc = lib.df11_decode(*bound, _stream_ptr(device))
    else:
        with torch.cuda.device(device):
            rc = lib.df11_decode(*bound, _stream_ptr(device))
    if rc:
        _native.check(rc, "df11_decode")
