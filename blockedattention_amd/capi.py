"""ctypes binding of the C ABI declared in include/blocked_attention.h.

Thin and explicit: torch tensors are used only as device memory (``data_ptr``)
and for the current HIP stream.  There is no CPU fallback: if the shared
library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libblockedattn_hip.so")

BA_F16, BA_BF16, BA_F32, BA_F64, BA_U8, BA_I8, BA_I16, BA_I32, BA_I64 = range(9)
META_FROM_LISTS, META_FROM_ACCUM, META_GIVEN = 0, 1, 2

SYMBOLS = (
    "ba_status_string", "ba_abi_version", "ba_plan_bytes", "ba_plan_gemm", "ba_plan_softmax", "ba_plan_read",
    "ba_plan_read_into", "ba_plan_gemm_notify", "ba_plan_softmax_notify", "ba_plan_wait",
    "ba_varlen_gemm", "ba_blocked_softmax", "ba_blocked_softmax_backward", "ba_gemm_softmax",
    "ba_varlen_attention", "ba_gemm_softmax_static", "ba_static_read", "ba_varlen_gemm_two",
)
MAILBOX_BYTES = 320
STATIC_MAX_SEGMENTS = 4096   # BA_STATIC_MAX_SEGMENTS


class PlanInfo(ctypes.Structure):
    _fields_ = [
        ("nseg", ctypes.c_int64), ("Dm1", ctypes.c_int64), ("Dm2", ctypes.c_int64), ("Dout", ctypes.c_int64),
        ("total_rows", ctypes.c_int64), ("gemm_items", ctypes.c_int64), ("strip_items", ctypes.c_int64),
        ("split_items", ctypes.c_int64), ("wide_items", ctypes.c_int64), ("pack_items", ctypes.c_int64),
        ("slow_items", ctypes.c_int64),
        ("max_M", ctypes.c_int32), ("max_N", ctypes.c_int32), ("max_K", ctypes.c_int32),
        ("bad_segments", ctypes.c_int32), ("run_errors", ctypes.c_int32), ("list_small", ctypes.c_int32), ("list_big", ctypes.c_int32), ("list_tile", ctypes.c_int32),
        ("list_rest", ctypes.c_int32), ("small_max_N", ctypes.c_int32), ("small_max_M", ctypes.c_int32),
        ("list_rows", ctypes.c_int32), ("att_blocks64", ctypes.c_int32), ("att_blocks128", ctypes.c_int32),
        ("list_mini", ctypes.c_int32), ("list_pipe", ctypes.c_int32), ("pipe_groups", ctypes.c_int32), ("min_N", ctypes.c_int32), ("min_K", ctypes.c_int32), ("ring_groups", ctypes.c_int32), ("wide_groups", ctypes.c_int32),
    ]

    def as_dict(self):
        return {name: getattr(self, name) for name, _ in self._fields_}


class BlockedAttentionError(RuntimeError):
    pass


_lib = None


def load():
    """Load libblockedattn_hip.so (built by ``python -m blockedattention_amd.build``)."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("BLOCKEDATTN_LIB", LIB_PATH)   # lets a caller point at another build of the library
    if not os.path.exists(path):
        raise BlockedAttentionError(
            f"{path} is missing: build it with `python -m blockedattention_amd.build lib` "
            "(there is no CPU or PyTorch fallback)")
    lib = ctypes.CDLL(path)
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    lib.ba_status_string.restype = ctypes.c_char_p
    lib.ba_status_string.argtypes = [i32]
    lib.ba_abi_version.restype = i32
    lib.ba_plan_bytes.restype = ctypes.c_size_t
    lib.ba_plan_bytes.argtypes = [i64]
    lib.ba_plan_gemm.restype = i32
    lib.ba_plan_gemm.argtypes = [vp, ctypes.c_size_t, i64, i32, vp, vp, vp, vp, vp, vp, vp]
    lib.ba_plan_softmax.restype = i32
    lib.ba_plan_softmax.argtypes = [vp, ctypes.c_size_t, i64, vp, vp, vp, i32, vp]
    lib.ba_plan_read.restype = i32
    lib.ba_plan_read.argtypes = [vp, ctypes.POINTER(PlanInfo), vp]
    u32 = ctypes.c_uint32
    lib.ba_plan_read_into.restype = i32
    lib.ba_plan_read_into.argtypes = [vp, ctypes.POINTER(PlanInfo), vp, vp]
    lib.ba_plan_gemm_notify.restype = i32
    lib.ba_plan_gemm_notify.argtypes = [vp, ctypes.c_size_t, i64, i32, vp, vp, vp, vp, vp, vp, vp, u32, vp]
    lib.ba_plan_softmax_notify.restype = i32
    lib.ba_plan_softmax_notify.argtypes = [vp, ctypes.c_size_t, i64, vp, vp, vp, i32, vp, u32, vp]
    lib.ba_plan_wait.restype = i32
    lib.ba_plan_wait.argtypes = [vp, u32, ctypes.POINTER(PlanInfo), i64]
    lib.ba_varlen_gemm.restype = i32
    lib.ba_varlen_gemm.argtypes = [vp, ctypes.POINTER(PlanInfo), i64, i32, vp, vp, vp, i64, i64, i64, i64, i32, i32, vp]
    lib.ba_blocked_softmax.restype = i32
    lib.ba_blocked_softmax.argtypes = [vp, ctypes.POINTER(PlanInfo), i64, i32, vp, vp, i64, i64, f32, vp]
    lib.ba_blocked_softmax_backward.restype = i32
    lib.ba_blocked_softmax_backward.argtypes = [vp, ctypes.POINTER(PlanInfo), i64, i32, vp, vp, vp, i64, i64, f32, vp]
    lib.ba_gemm_softmax.restype = i32
    lib.ba_gemm_softmax.argtypes = [vp, ctypes.POINTER(PlanInfo), i64, i32, vp, vp, vp, i32, i64, i64, i64, i64, f32, vp]
    lib.ba_varlen_attention.restype = i32
    lib.ba_varlen_attention.argtypes = [vp, ctypes.POINTER(PlanInfo), i64, i32, vp, vp, vp, vp, i64, i64, i64, i64, f32, vp]
    lib.ba_gemm_softmax_static.restype = i32
    lib.ba_gemm_softmax_static.argtypes = [i64, i32, vp, vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, i64, i64, i64, i64, f32, vp]
    lib.ba_static_read.restype = i32
    lib.ba_static_read.argtypes = [vp, vp]
    lib.ba_varlen_gemm_two.restype = i32
    lib.ba_varlen_gemm_two.argtypes = [i32, i64, vp, ctypes.POINTER(PlanInfo), vp, vp, vp, i64, i64, i64,
                                       vp, ctypes.POINTER(PlanInfo), vp, vp, vp, i64, i64, i64, vp]
    _lib = lib
    return lib


def check(status, what):
    if status != 0:
        raise BlockedAttentionError(f"{what}: {load().ba_status_string(status).decode()} (status {status})")


def dtype_code(dtype):
    try:
        return {torch.float16: BA_F16, torch.bfloat16: BA_BF16, torch.float32: BA_F32, torch.float64: BA_F64,
                torch.uint8: BA_U8, torch.int8: BA_I8, torch.int16: BA_I16, torch.int32: BA_I32,
                torch.int64: BA_I64}[dtype]
    except KeyError:
        raise BlockedAttentionError(f"unsupported dtype {dtype}") from None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _meta(t, n, name):
    if t is None:
        return None
    if t.dtype != torch.int64 or not t.is_cuda or not t.is_contiguous() or t.numel() != n:
        raise BlockedAttentionError(f"{name} must be a contiguous int64 device tensor with {n} entries")
    return t


class Plan:
    """Device-resident schedule for one batch of segments (see ba_plan_gemm / ba_plan_softmax)."""

    def __init__(self, nseg, device):
        self.nseg = int(nseg)
        self.bytes = load().ba_plan_bytes(self.nseg)
        self.buf = torch.empty(self.bytes, dtype=torch.uint8, device=device)
        self.info = None

    @property
    def ptr(self):
        return ctypes.c_void_p(self.buf.data_ptr())

    def read(self, raise_on_bad=True):
        """Blocking: copy the plan summary to the host (and remember it as the launch hint)."""
        info = PlanInfo()
        st = load().ba_plan_read(self.ptr, ctypes.byref(info), _stream())
        if st != 0 and (raise_on_bad or st != 5):
            check(st, "ba_plan_read")
        self.info = info
        return info

    def read_into(self, staging, raise_on_bad=True):
        """As read(), the summary travelling through `staging` (a pinned CPU tensor of at least 256 bytes)."""
        info = PlanInfo()
        st = load().ba_plan_read_into(self.ptr, ctypes.byref(info), ctypes.c_void_p(staging.data_ptr()), _stream())
        if st != 0 and (raise_on_bad or st != 5):
            check(st, "ba_plan_read_into")
        self.info = info
        return info

    def wait(self, mailbox, ticket, timeout_us=10_000_000, raise_on_bad=True):
        """The summary a *_notify scheduler call wrote into `mailbox` (pinned CPU tensor): spins on the host, no
        copy and no stream synchronisation."""
        info = PlanInfo()
        st = load().ba_plan_wait(ctypes.c_void_p(mailbox.data_ptr()), ticket, ctypes.byref(info), timeout_us)
        if st != 0 and (raise_on_bad or st != 5):
            check(st, "ba_plan_wait")
        self.info = info
        return info

    def _hint(self):
        return ctypes.byref(self.info) if self.info is not None else None


def plan_gemm(nseg, device, MList=None, NList=None, KList=None, accum1=None, accum2=None, accumOut=None,
              mode=None, plan=None, mailbox=None, ticket=0):
    """Run the scheduler.  Tensors passed as None in an *output* role are not written.

    ``plan``: an existing Plan of the same segment count to schedule into again (no allocation, e.g.
    under stream capture); its host summary is dropped, since it describes the previous schedule.
    ``mailbox`` (pinned CPU tensor of MAILBOX_BYTES) and ``ticket``: the scheduler also hands the summary to the
    host there; collect it with ``plan.wait(mailbox, ticket)``."""
    have_lists = MList is not None and NList is not None and KList is not None
    have_accum = accum1 is not None and accum2 is not None and accumOut is not None
    if mode is None:
        mode = META_GIVEN if (have_lists and have_accum) else (META_FROM_LISTS if have_lists else META_FROM_ACCUM)
    for t, n, name in ((MList, nseg, "MList"), (NList, nseg, "NList"), (KList, nseg, "KList"),
                       (accum1, nseg + 1, "mat1Accum"), (accum2, nseg + 1, "mat2Accum"),
                       (accumOut, nseg + 1, "outAccum")):
        _meta(t, n, name)
    if plan is None:
        plan = Plan(nseg, device)
    elif plan.nseg != int(nseg):
        raise BlockedAttentionError(f"the plan was sized for {plan.nseg} segments, not {nseg}")
    plan.info = None
    if mailbox is not None:
        st = load().ba_plan_gemm_notify(plan.ptr, plan.bytes, nseg, mode, _ptr(MList), _ptr(NList), _ptr(KList),
                                        _ptr(accum1), _ptr(accum2), _ptr(accumOut), ctypes.c_void_p(mailbox.data_ptr()),
                                        ticket, _stream())
        check(st, "ba_plan_gemm_notify")
        return plan
    st = load().ba_plan_gemm(plan.ptr, plan.bytes, nseg, mode, _ptr(MList), _ptr(NList), _ptr(KList),
                             _ptr(accum1), _ptr(accum2), _ptr(accumOut), _stream())
    check(st, "ba_plan_gemm")
    return plan


def plan_softmax(nseg, device, rowList, colList, accum=None, accum_given=False):
    _meta(rowList, nseg, "rowList"); _meta(colList, nseg, "colList"); _meta(accum, nseg + 1, "srcAccum")
    plan = Plan(nseg, device)
    st = load().ba_plan_softmax(plan.ptr, plan.bytes, nseg, _ptr(rowList), _ptr(colList), _ptr(accum),
                                int(bool(accum_given)), _stream())
    check(st, "ba_plan_softmax")
    return plan


def varlen_gemm(plan, A, B, out, H, Dm1, Dm2, Dout, transpose1=False, transpose2=False):
    st = load().ba_varlen_gemm(plan.ptr, plan._hint(), plan.nseg, dtype_code(A.dtype), _ptr(A), _ptr(B), _ptr(out), H, Dm1, Dm2,
                               Dout, int(transpose1), int(transpose2), _stream())
    check(st, "ba_varlen_gemm")
    return out


def blocked_softmax(plan, src, dst, H, Dsrc, scale=1.0):
    st = load().ba_blocked_softmax(plan.ptr, plan._hint(), plan.nseg, dtype_code(src.dtype), _ptr(src), _ptr(dst), H, Dsrc,
                                   float(scale), _stream())
    check(st, "ba_blocked_softmax")
    return dst


def blocked_softmax_backward(plan, y, dy, dx, H, Dsrc, scale=1.0):
    st = load().ba_blocked_softmax_backward(plan.ptr, plan._hint(), plan.nseg, dtype_code(y.dtype), _ptr(y), _ptr(dy), _ptr(dx),
                                            H, Dsrc, float(scale), _stream())
    check(st, "ba_blocked_softmax_backward")
    return dx


def gemm_softmax(plan, A, B, out, H, Dm1, Dm2, Dout, scale=1.0):
    st = load().ba_gemm_softmax(plan.ptr, plan._hint(), plan.nseg, dtype_code(A.dtype), _ptr(A), _ptr(B), _ptr(out),
                                dtype_code(out.dtype), H, Dm1, Dm2, Dout, float(scale), _stream())
    check(st, "ba_gemm_softmax")
    return out


def gemm_softmax_static(MList, NList, KList, A, B, out, H, Dm1, Dm2, Dout, scale=1.0, accum1=None, accum2=None,
                        accumOut=None, mode=META_FROM_LISTS):
    """Scheduler + fused pair with the plan in the library's own device buffer (see ba_gemm_softmax_static):
    no allocation, no read-back."""
    nseg = MList.numel() if MList is not None else accumOut.numel() - 1
    st = load().ba_gemm_softmax_static(nseg, mode, _ptr(MList), _ptr(NList), _ptr(KList), _ptr(accum1), _ptr(accum2),
                                       _ptr(accumOut), dtype_code(A.dtype), _ptr(A), _ptr(B), _ptr(out),
                                       dtype_code(out.dtype), H, Dm1, Dm2, Dout, float(scale), _stream())
    check(st, "ba_gemm_softmax_static")
    return out


def varlen_gemm_two(plan_a, A_a, B_a, out_a, dims_a, plan_b, A_b, B_b, out_b, dims_b, H):
    """Both products as one launch (see ba_varlen_gemm_two); False where the library wants two calls instead."""
    st = load().ba_varlen_gemm_two(dtype_code(A_a.dtype), H, plan_a.ptr, plan_a._hint(), _ptr(A_a), _ptr(B_a), _ptr(out_a), *dims_a,
                                   plan_b.ptr, plan_b._hint(), _ptr(A_b), _ptr(B_b), _ptr(out_b), *dims_b, _stream())
    if st == 3:
        return False
    check(st, "ba_varlen_gemm_two")
    return True


def static_read(raise_on_bad=True):
    """Summary of the last gemm_softmax_static call on the current stream (see ba_static_read)."""
    info = PlanInfo()
    st = load().ba_static_read(ctypes.byref(info), _stream())
    if st != 0 and (raise_on_bad or st != 5):
        check(st, "ba_static_read")
    return info, st


def varlen_attention(plan, Q, K, V, out, H, Dm1, Dm2, Dout, scale=1.0):
    """out [H, Dm1] <- softmax(scale * Q_g K_g^T) V_g per segment (see ba_varlen_attention)."""
    st = load().ba_varlen_attention(plan.ptr, plan._hint(), plan.nseg, dtype_code(Q.dtype), _ptr(Q), _ptr(K), _ptr(V),
                                    _ptr(out), H, Dm1, Dm2, Dout, float(scale), _stream())
    check(st, "ba_varlen_attention")
    return out
