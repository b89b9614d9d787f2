"""ctypes binding of the C ABI in ``include/ts_hip.h`` (``libts_hip.so``).

Kernel-level entry points on flattened ``[B, E|N, K]`` buffers. PyTorch is used
only to own device memory and to name the stream; every call launches on the
current stream of the tensors' device and never synchronises. The library must
have been built (``python -c "import __graft_entry__ as g; g.build()"`` or
``make -C pytorch_scatter_amd/csrc``): there is no fallback path.
"""
import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TS_HIP_LIB", os.path.join(_HERE, "libts_hip.so"))  # env: tuning aid

SUM, MEAN, MUL, DIV, MIN, MAX = range(6)
REDUCE = {"sum": SUM, "add": SUM, "mean": MEAN, "mul": MUL, "min": MIN, "max": MAX}
DTYPE = {torch.float32: 0, torch.float64: 1, torch.float16: 2, torch.bfloat16: 3,
         torch.int32: 4, torch.int64: 5, torch.int16: 6, torch.int8: 7, torch.uint8: 8}

EXPORTS = (
    "ts_error_string", "ts_hip_version", "ts_status_gave_up", "ts_selftest_lane_ops", "ts_scatter_last_route", "ts_scatter_route_name",
    "ts_segment_csr_workspace_bytes", "ts_segment_csr", "ts_segment_csr_static", "ts_gather_csr",
    "ts_segment_mean_csr_backward",
    "ts_segment_coo_workspace_bytes", "ts_segment_coo", "ts_gather_coo",
    "ts_segment_mean_coo_backward",
    "ts_scatter", "ts_scatter_workspace_bytes", "ts_scatter_workspace_zero_bytes", "ts_scatter_with_workspace", "ts_scatter_count", "ts_scatter_count_workspace_bytes", "ts_scatter_count_with_workspace", "ts_scatter_sum_count_workspace_bytes", "ts_scatter_sum_count_with_workspace", "ts_divide_by_count", "ts_arg_backward",
    "ts_group_softmax_workspace_bytes", "ts_group_softmax", "ts_group_softmax_backward",
    "ts_group_logsumexp", "ts_group_logsumexp_backward",
    "ts_group_std", "ts_group_std_backward", "ts_group_bins_workspace_bytes", "ts_group_workspace_bytes", "ts_group_std_forward",
    "ts_group_std_backward_with_workspace", "ts_group_logsumexp_backward_with_workspace",
    "ts_index_to_indptr", "ts_indptr_to_index_workspace_bytes", "ts_indptr_to_index",
    "ts_sort_index_workspace_bytes", "ts_sort_index",
    "ts_segment_csr_permuted_workspace_bytes", "ts_segment_csr_permuted",
)

_lib = None


class TsError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: the HIP kernels are not built "
                "(run `make -C pytorch_scatter_amd/csrc -j8`); there is no CPU fallback")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.ts_error_string.restype = ctypes.c_char_p
        _lib.ts_hip_version.restype = ctypes.c_int64
        _lib.ts_segment_csr_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_segment_coo_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_group_softmax_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_indptr_to_index_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_scatter_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_scatter_workspace_zero_bytes.restype = ctypes.c_size_t
        _lib.ts_scatter_count_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_scatter_sum_count_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_sort_index_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_group_bins_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_group_workspace_bytes.restype = ctypes.c_size_t
        _lib.ts_segment_csr_permuted_workspace_bytes.restype = ctypes.c_size_t
    return _lib


def _check(rc: int):
    if rc != 0:
        raise TsError(f"ts_hip: {lib().ts_error_string(rc).decode()} (status {rc})")


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i(v):
    return ctypes.c_int64(int(v))


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise TsError("ts_hip: all buffers must be device (HIP) tensors")


STATUS_BYTES = 256  # TS_STATUS_BYTES of include/ts_hip.h
# Set (TS_CHECK_STATUS=1, as the GPU tests do): the segment wrappers below wait for the stream and raise if the
# call's status word is not 0, i.e. if a row was given up by the look-back.
CHECK_STATUS = os.environ.get("TS_CHECK_STATUS") == "1"


def status_word(ws: torch.Tensor, nbytes: int) -> int:
    """1 if the latest segment reduction that used `ws` gave a row up, else 0 (waits for the device): the two
    status words hold the tag of the latest call and the tag of the latest call that gave a row up."""
    call, gave_up = ws[nbytes - STATUS_BYTES:nbytes - STATUS_BYTES + 16].view(torch.int64).tolist()
    return int(call != 0 and gave_up == call)


def _check_status(ws, nbytes, B, N, K):
    if CHECK_STATUS and nbytes >= STATUS_BYTES and B * N * K > 0:
        word = status_word(ws, nbytes)
        if word != 0:
            raise TsError(f"ts_hip: segment reduction left status word {word}: a row was given up")


def scatter_last_route() -> str:
    """Name of the kernels the last scatter call of this thread launched (ts_scatter_last_route)."""
    L = lib()
    L.ts_scatter_route_name.restype = ctypes.c_char_p
    return L.ts_scatter_route_name(L.ts_scatter_last_route()).decode()


def hip_version() -> int:
    return int(lib().ts_hip_version())


def segment_csr(src, indptr, out, arg_out, B, N, E, K, indptr_batch_stride, reduce: int):
    _dev(src, indptr, out, arg_out)
    L = lib()
    nbytes = L.ts_segment_csr_workspace_bytes(_i(B), _i(N), _i(E), _i(K), DTYPE[out.dtype], reduce)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(L.ts_segment_csr(_p(src), _p(indptr), _p(out), _p(arg_out), _i(B), _i(N), _i(E), _i(K),
                                _i(indptr_batch_stride), DTYPE[out.dtype], reduce, _p(ws),
                                ctypes.c_size_t(nbytes), _stream(out)))
    _check_status(ws, nbytes, B, N, K)
    return ws


STATIC_SCRATCH_BYTES = 8 << 20  # TS_STATIC_SCRATCH_BYTES of include/ts_hip.h


def segment_csr_static(src, indptr, out, arg_out, B, N, E, K, indptr_batch_stride, reduce: int):
    """ts_segment_csr_static: the same reduction with the library's own device array as scratch; nothing is
    allocated here or in the library. Raises TsError (workspace) for inputs beyond the array's size."""
    _dev(src, indptr, out, arg_out)
    with torch.cuda.device(out.device):
        _check(lib().ts_segment_csr_static(_p(src), _p(indptr), _p(out), _p(arg_out), _i(B), _i(N), _i(E), _i(K),
                                           _i(indptr_batch_stride), DTYPE[out.dtype], reduce, _stream(out)))


def gather_csr(src, indptr, out, B, N, E, K, indptr_batch_stride):
    _dev(src, indptr, out)
    with torch.cuda.device(out.device):
        _check(lib().ts_gather_csr(_p(src), _p(indptr), _p(out), _i(B), _i(N), _i(E), _i(K),
                                   _i(indptr_batch_stride), DTYPE[out.dtype], _stream(out)))


def segment_mean_csr_backward(grad_out, indptr, grad_in, B, N, E, K, indptr_batch_stride):
    _dev(grad_out, indptr, grad_in)
    with torch.cuda.device(grad_in.device):
        _check(lib().ts_segment_mean_csr_backward(_p(grad_out), _p(indptr), _p(grad_in), _i(B), _i(N),
                                                  _i(E), _i(K), _i(indptr_batch_stride),
                                                  DTYPE[grad_in.dtype], _stream(grad_in)))


def segment_coo(src, index, out, arg_out, count_out, B, N, E, K, index_batch_stride, reduce: int,
                out_given: bool):
    _dev(src, index, out, arg_out, count_out)
    L = lib()
    nbytes = L.ts_segment_coo_workspace_bytes(_i(B), _i(N), _i(E), _i(K), DTYPE[out.dtype], reduce)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(L.ts_segment_coo(_p(src), _p(index), _p(out), _p(arg_out), _p(count_out), _i(B), _i(N),
                                _i(E), _i(K), _i(index_batch_stride), DTYPE[out.dtype], reduce,
                                int(out_given), _p(ws), ctypes.c_size_t(nbytes), _stream(out)))
    _check_status(ws, nbytes, B, N, K)
    return ws


def gather_coo(src, index, out, B, N, E, K, index_batch_stride):
    _dev(src, index, out)
    with torch.cuda.device(out.device):
        _check(lib().ts_gather_coo(_p(src), _p(index), _p(out), _i(B), _i(N), _i(E), _i(K),
                                   _i(index_batch_stride), DTYPE[out.dtype], _stream(out)))


def segment_mean_coo_backward(grad_out, index, count, grad_in, B, N, E, K, index_batch_stride):
    _dev(grad_out, index, count, grad_in)
    with torch.cuda.device(grad_in.device):
        _check(lib().ts_segment_mean_coo_backward(_p(grad_out), _p(index), _p(count), _p(grad_in), _i(B),
                                                  _i(N), _i(E), _i(K), _i(index_batch_stride),
                                                  DTYPE[grad_in.dtype], _stream(grad_in)))


def scatter(src, index, out, arg_out, B, E, K, N, sb, se, sk, reduce: int, out_given: bool):
    _dev(src, index, out, arg_out)
    with torch.cuda.device(out.device):
        _check(lib().ts_scatter(_p(src), _p(index), _p(out), _p(arg_out), _i(B), _i(E), _i(K), _i(N),
                                _i(sb), _i(se), _i(sk), DTYPE[out.dtype], reduce, int(out_given),
                                _stream(out)))


def scatter_with_workspace(src, index, out, arg_out, B, E, K, N, sb, se, sk, reduce: int, out_given: bool, ws=None):
    _dev(src, index, out, arg_out)
    L = lib()
    nbytes = L.ts_scatter_workspace_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[out.dtype], reduce)
    nzero = L.ts_scatter_workspace_zero_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[out.dtype], reduce)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
        ws[:nzero].zero_()  # the part that has to read as zero; the call leaves it zero for the next one
    with torch.cuda.device(out.device):
        _check(L.ts_scatter_with_workspace(_p(src), _p(index), _p(out), _p(arg_out), _i(B), _i(E), _i(K), _i(N),
                                           _i(sb), _i(se), _i(sk), DTYPE[out.dtype], reduce, int(out_given),
                                           _p(ws) if nbytes else None, ctypes.c_size_t(nbytes), _stream(out)))
    if CHECK_STATUS and nzero >= STATUS_BYTES:
        # min / max of single values: the word behind the key table is set when a bounded wait in the kernel ran out
        if int(ws[nzero - STATUS_BYTES:nzero - STATUS_BYTES + 8].view(torch.int64).item()) != 0:
            raise TsError("ts_hip: scatter min / max lost entries: a bounded wait inside the kernel ran out")
    return ws


def scatter_count(index, count, B, E, N, sb, se):
    _dev(index, count)
    with torch.cuda.device(count.device):
        _check(lib().ts_scatter_count(_p(index), _p(count), _i(B), _i(E), _i(N), _i(sb), _i(se),
                                      _stream(count)))


def scatter_count_with_workspace(index, count, B, E, N, sb, se):
    _dev(index, count)
    L = lib()
    nbytes = L.ts_scatter_count_workspace_bytes(_i(B), _i(E), _i(N))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=count.device)
    with torch.cuda.device(count.device):
        _check(L.ts_scatter_count_with_workspace(_p(index), _p(count), _i(B), _i(E), _i(N), _i(sb), _i(se),
                                                 _p(ws) if nbytes else None, ctypes.c_size_t(nbytes), _stream(count)))
    return nbytes


def scatter_sum_count_with_workspace(src, index, out, count, B, E, K, N, sb, se, out_given: bool):
    """Sum and int32 count of the entries per output row in one call (ts_scatter_sum_count_with_workspace)."""
    _dev(src, index, out, count)
    L = lib()
    nbytes = L.ts_scatter_sum_count_workspace_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[out.dtype])
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(L.ts_scatter_sum_count_with_workspace(_p(src), _p(index), _p(out), _p(count), _i(B), _i(E), _i(K), _i(N),
                                                     _i(sb), _i(se), DTYPE[out.dtype], 1 if out_given else 0,
                                                     _p(ws) if nbytes else None, ctypes.c_size_t(nbytes), _stream(out)))
    return nbytes


def divide_by_count(out, count, B, N, K):
    _dev(out, count)
    with torch.cuda.device(out.device):
        _check(lib().ts_divide_by_count(_p(out), _p(count), _i(B), _i(N), _i(K), DTYPE[out.dtype],
                                        _stream(out)))


def arg_backward(grad_out, arg, grad_in, B, N, E, K):
    _dev(grad_out, arg, grad_in)
    with torch.cuda.device(grad_in.device):
        _check(lib().ts_arg_backward(_p(grad_out), _p(arg), _p(grad_in), _i(B), _i(N), _i(E), _i(K),
                                     DTYPE[grad_in.dtype], _stream(grad_in)))


def _group_workspace(like, B, N, K):
    nbytes = lib().ts_group_softmax_workspace_bytes(_i(B), _i(N), _i(K), DTYPE[like.dtype])
    return torch.empty(max(nbytes, 1), dtype=torch.uint8, device=like.device), nbytes


def group_bins_workspace_bytes(B, E, K, N, dtype) -> int:
    """Scratch of the route through buckets of groups (ts_group_bins_workspace_bytes); 0: the route does not apply."""
    return int(lib().ts_group_bins_workspace_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[dtype]))


def group_softmax(src, index, out, B, E, K, N, sb, se, log_space: bool, eps: float = 1e-12):
    _dev(src, index, out)
    # the workspace that opens every route: three passes, buckets of groups (unsorted index), one-pass tiles (sorted)
    nbytes = int(lib().ts_group_workspace_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[out.dtype]))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(lib().ts_group_softmax(_p(src), _p(index), _p(out), _i(B), _i(E), _i(K), _i(N), _i(sb), _i(se),
                                      DTYPE[out.dtype], int(log_space), ctypes.c_double(eps), _p(ws),
                                      ctypes.c_size_t(nbytes), _stream(out)))
    return ws


def group_softmax_backward(result, grad_out, index, grad_in, B, E, K, N, sb, se, log_space: bool):
    _dev(result, grad_out, index, grad_in)
    nbytes = int(lib().ts_group_workspace_bytes(_i(B), _i(E), _i(K), _i(N), DTYPE[grad_in.dtype]))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=grad_in.device)
    with torch.cuda.device(grad_in.device):
        _check(lib().ts_group_softmax_backward(_p(result), _p(grad_out), _p(index), _p(grad_in), _i(B), _i(E),
                                               _i(K), _i(N), _i(sb), _i(se), DTYPE[grad_in.dtype],
                                               int(log_space), _p(ws), ctypes.c_size_t(nbytes),
                                               _stream(grad_in)))
    return ws


def group_logsumexp(src, index, out, B, E, K, N, sb, se, eps: float = 1e-12, bins: bool = True):
    """bins: hand over the larger workspace with which the call goes through buckets of groups where that applies."""
    _dev(src, index, out)
    ws, nbytes = _group_workspace(out, B, N, K)
    big = group_bins_workspace_bytes(B, E, K, N, out.dtype) if bins else 0
    if big > nbytes:
        nbytes = big
        ws = torch.empty(nbytes, dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(lib().ts_group_logsumexp(_p(src), _p(index), _p(out), _i(B), _i(E), _i(K), _i(N), _i(sb), _i(se),
                                        DTYPE[out.dtype], ctypes.c_double(eps), _p(ws), ctypes.c_size_t(nbytes),
                                        _stream(out)))
    return ws


def group_logsumexp_backward(src, index, out, grad_out, grad_in, B, E, K, N, sb, se, with_workspace: bool = True):
    _dev(src, index, out, grad_out, grad_in)
    with torch.cuda.device(grad_in.device):
        if with_workspace:
            ws, nbytes = _group_workspace(grad_in, B, N, K)
            _check(lib().ts_group_logsumexp_backward_with_workspace(
                _p(src), _p(index), _p(out), _p(grad_out), _p(grad_in), _i(B), _i(E), _i(K), _i(N), _i(sb), _i(se),
                DTYPE[grad_in.dtype], _p(ws), ctypes.c_size_t(nbytes), _stream(grad_in)))
        else:
            _check(lib().ts_group_logsumexp_backward(_p(src), _p(index), _p(out), _p(grad_out), _p(grad_in), _i(B),
                                                     _i(E), _i(K), _i(N), _i(sb), _i(se), DTYPE[grad_in.dtype],
                                                     _stream(grad_in)))


def group_std(src, index, total, count, out, B, E, K, N, sb, se, unbiased: bool = True):
    _dev(src, index, total, count, out)
    ws, nbytes = _group_workspace(out, B, N, K)
    with torch.cuda.device(out.device):
        _check(lib().ts_group_std(_p(src), _p(index), _p(total), _p(count), _p(out), _i(B), _i(E), _i(K), _i(N),
                                  _i(sb), _i(se), DTYPE[out.dtype], int(unbiased), _p(ws), ctypes.c_size_t(nbytes),
                                  _stream(out)))
    return ws


def group_std_forward(src, index, total, count, out, B, E, K, N, sb, se, unbiased: bool = True):
    """Group sums, counts and standard deviation in one call through buckets of groups (ts_group_std_forward).
    Returns the bytes of workspace used; raises where the route does not apply."""
    _dev(src, index, total, count, out)
    nbytes = group_bins_workspace_bytes(B, E, K, N, out.dtype)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(lib().ts_group_std_forward(_p(src), _p(index), _p(total), _p(count), _p(out), _i(B), _i(E), _i(K), _i(N),
                                          _i(sb), _i(se), DTYPE[out.dtype], int(unbiased), _p(ws),
                                          ctypes.c_size_t(nbytes), _stream(out)))
    return nbytes


def group_std_backward(src, index, total, count, out, grad_out, grad_in, B, E, K, N, sb, se, unbiased: bool = True,
                       with_workspace: bool = True):
    _dev(src, index, total, count, out, grad_out, grad_in)
    with torch.cuda.device(grad_in.device):
        if with_workspace:
            ws, nbytes = _group_workspace(grad_in, B, N, K)
            _check(lib().ts_group_std_backward_with_workspace(
                _p(src), _p(index), _p(total), _p(count), _p(out), _p(grad_out), _p(grad_in), _i(B), _i(E), _i(K), _i(N),
                _i(sb), _i(se), DTYPE[grad_in.dtype], int(unbiased), _p(ws), ctypes.c_size_t(nbytes), _stream(grad_in)))
        else:
            _check(lib().ts_group_std_backward(_p(src), _p(index), _p(total), _p(count), _p(out), _p(grad_out),
                                               _p(grad_in), _i(B), _i(E), _i(K), _i(N), _i(sb), _i(se),
                                               DTYPE[grad_in.dtype], int(unbiased), _stream(grad_in)))


def index_to_indptr(index, indptr, B, E, N, index_batch_stride):
    _dev(index, indptr)
    with torch.cuda.device(indptr.device):
        _check(lib().ts_index_to_indptr(_p(index), _p(indptr), _i(B), _i(E), _i(N), _i(index_batch_stride),
                                        _stream(indptr)))


def indptr_to_index(indptr, index, B, N, E, indptr_batch_stride):
    _dev(indptr, index)
    L = lib()
    nbytes = L.ts_indptr_to_index_workspace_bytes(_i(B), _i(N))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=index.device)
    with torch.cuda.device(index.device):
        _check(L.ts_indptr_to_index(_p(indptr), _p(index), _i(B), _i(N), _i(E), _i(indptr_batch_stride), _p(ws),
                                    ctypes.c_size_t(nbytes), _stream(index)))
    return ws


def sort_index(index, perm, indptr, E, N):
    _dev(index, perm, indptr)
    L = lib()
    with torch.cuda.device(indptr.device):
        nbytes = L.ts_sort_index_workspace_bytes(_i(E), _i(N))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=indptr.device)
        _check(L.ts_sort_index(_p(index), _p(perm), _p(indptr), _i(E), _i(N), _p(ws), ctypes.c_size_t(nbytes),
                               _stream(indptr)))
    return ws


def segment_csr_permuted(src, perm, indptr, out, arg_out, B, N, E, K, perm_batch_stride, indptr_batch_stride,
                         reduce: int):
    _dev(src, perm, indptr, out, arg_out)
    L = lib()
    nbytes = L.ts_segment_csr_permuted_workspace_bytes(_i(B), _i(N), _i(E), _i(K), DTYPE[out.dtype], reduce)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=out.device)
    with torch.cuda.device(out.device):
        _check(L.ts_segment_csr_permuted(_p(src), _p(perm), _p(indptr), _p(out), _p(arg_out), _i(B), _i(N), _i(E),
                                         _i(K), _i(perm_batch_stride), _i(indptr_batch_stride), DTYPE[out.dtype],
                                         reduce, _p(ws), ctypes.c_size_t(nbytes), _stream(out)))
    _check_status(ws, nbytes, B, N, K)
    return ws
