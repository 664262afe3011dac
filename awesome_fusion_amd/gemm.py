"""ctypes binding of the C ABI in include/bfaintb_gemm.h.

Arguments mirror the reference's launch block {c, a, b, scale, m, n, k, lda, ldb, ldc}
(/root/reference/bfAintBGemm/bfAintBGemm.cc:119-133).  Tensors are only carriers of device
pointers (``data_ptr()``); torch supplies device memory and streams, nothing else.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libbfaintb_gemm.so")

AUTO, DECODE, PREFILL = 0, 1, 2
PREFILL_256, PREFILL_128 = 3, 4  # the tiled variant with its tile size forced (tests, tuning)
PREFILL_256_LDS = 5               # ... and its form with both operands in LDS forced
PREFILL_128_LDS = 6               # the same for the 128-tile kernel
PREFILL_256X128 = 7               # tiles of 256 rows x 128 columns, weights in registers
ACT_NONE, ACT_SILU_GATE = 0, 1


class BfaintbError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what} failed: [{code}] {error_string(code)}")


def library_path():
    return _LIB


def build_library(verbose=False):
    """Compile every HIP source for gfx950 into libbfaintb_gemm.so (hipcc cross-compiles without a GPU)."""
    global _lib
    r = subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-B", "-j8"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:])
        print(r.stderr[-4000:])
    if r.returncode != 0:
        raise RuntimeError("building libbfaintb_gemm.so failed")
    _lib = None


_lib = None
_u32 = C.c_uint32
_vp = C.c_void_p


class Epilogue(C.Structure):
    """bfaintb_epilogue of include/bfaintb_gemm.h."""
    _fields_ = [("bias", C.c_void_p), ("residual", C.c_void_p), ("ldr", C.c_uint32), ("activation", C.c_uint32)]


class PackedHeader(C.Structure):
    """bfaintb_packed_header of include/bfaintb_gemm.h: the 64-byte header of a pre-packed weight file."""
    _fields_ = [("magic", C.c_char * 8), ("header_bytes", _u32), ("layout", _u32), ("weight_bits", _u32), ("group_size", _u32),
                ("k", _u32), ("n", _u32), ("payload_bytes", C.c_uint64), ("scale_bytes", C.c_uint64), ("has_bias", _u32),
                ("reserved", _u32 * 3)]


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise RuntimeError(
                f"{_LIB} is missing: build it with `make -C awesome_fusion_amd/csrc` "
                "(or __graft_entry__.build()); this package has no CPU fallback")
        # torch ships its own HIP runtime: when a process is going to use torch for device memory (this binding's callers
        # do), that runtime has to be the one this library binds to, so torch is loaded first.  Loaded the other way round,
        # the library's launches fail with "no ROCm-capable device" against tensors torch allocated.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(_LIB)
        L.bfaintb_gemm.restype = C.c_int
        L.bfaintb_gemm.argtypes = [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp,
                                   C.c_size_t, _vp]
        L.bfaintb_gemm_ex.restype = C.c_int
        L.bfaintb_gemm_ex.argtypes = L.bfaintb_gemm.argtypes + [C.c_int, _u32]
        L.bfaintb_gemm_bias.restype = C.c_int
        L.bfaintb_gemm_bias.argtypes = [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp,
                                        C.c_size_t, _vp]
        L.bfaintb_gemm_fused.restype = C.c_int
        L.bfaintb_gemm_fused.argtypes = [_vp, _vp, _vp, _vp, C.POINTER(Epilogue), _u32, _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp,
                                         C.c_size_t, _vp]
        L.bfaintb_gemm_prepacked_fused.restype = C.c_int
        L.bfaintb_gemm_prepacked_fused.argtypes = [_vp, _vp, _vp, _vp, C.POINTER(Epilogue), _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp,
                                                   C.c_size_t, _vp]
        L.bfaintb_gemm_reference.restype = C.c_int
        L.bfaintb_gemm_reference.argtypes = [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _vp, C.c_size_t, _vp]
        L.bfaintb_gemm_reference_ex.restype = C.c_int
        L.bfaintb_gemm_reference_ex.argtypes = L.bfaintb_gemm_reference.argtypes + [C.c_int, _u32]
        L.bfaintb_gemm_workspace_bytes.restype = C.c_size_t
        L.bfaintb_gemm_workspace_bytes.argtypes = [_u32, _u32, _u32, C.c_int, _u32]
        L.bfaintb_gemm_workspace_bytes_ex.restype = C.c_size_t
        L.bfaintb_gemm_workspace_bytes_ex.argtypes = [_u32, _u32, _u32, C.c_int, _u32, C.c_int, _u32]
        L.bfaintb_workspace_init.restype = C.c_int
        L.bfaintb_workspace_init.argtypes = [_vp, C.c_size_t, _vp]
        L.bfaintb_gemm_variant.restype = C.c_int
        L.bfaintb_gemm_variant.argtypes = [_u32, _u32, _u32, C.c_int, _u32]
        L.bfaintb_gemm_split_k.restype = _u32
        L.bfaintb_gemm_split_k.argtypes = [_u32, _u32, _u32, C.c_int, _u32]
        L.bfaintb_prepack_bytes.restype = C.c_size_t
        L.bfaintb_prepack_bytes.argtypes = [_u32, _u32, C.c_int]
        L.bfaintb_prepack.restype = C.c_int
        L.bfaintb_prepack.argtypes = [_vp, _vp, _u32, _u32, _u32, C.c_int, _vp]
        L.bfaintb_prepack_colmajor.restype = C.c_int
        L.bfaintb_prepack_colmajor.argtypes = [_vp, _vp, _u32, _u32, _u32, C.c_int, _vp]
        L.bfaintb_unpack.restype = C.c_int
        L.bfaintb_unpack.argtypes = [_vp, _vp, _u32, _u32, _u32, C.c_int, _vp]
        L.bfaintb_gemm_prepacked.restype = C.c_int
        L.bfaintb_gemm_prepacked.argtypes = [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp, C.c_size_t, _vp]
        L.bfaintb_gemm_prepacked_workspace_bytes_ex.restype = C.c_size_t
        L.bfaintb_gemm_prepacked_workspace_bytes_ex.argtypes = [_u32, _u32, _u32, C.c_int, _u32, C.c_int]
        L.bfaintb_gemm_prepacked_ex.restype = C.c_int
        L.bfaintb_gemm_prepacked_ex.argtypes = L.bfaintb_gemm_prepacked.argtypes + [C.c_int]
        L.bfaintb_gemm_prepacked_variant.restype = C.c_int
        L.bfaintb_gemm_prepacked_variant.argtypes = [_u32, _u32, _u32, C.c_int, _u32]
        L.bfaintb_packed_header_init.restype = C.c_int
        L.bfaintb_packed_header_init.argtypes = [C.POINTER(PackedHeader), _u32, _u32, C.c_int, _u32, C.c_int]
        L.bfaintb_packed_header_check.restype = C.c_int
        L.bfaintb_packed_header_check.argtypes = [C.POINTER(PackedHeader)]
        L.bfaintb_dequant.restype = C.c_int
        L.bfaintb_dequant.argtypes = [_vp, _vp, _vp, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp]
        L.bfaintb_probe_read.restype = C.c_int
        L.bfaintb_probe_read.argtypes = [_vp, C.c_size_t, _vp, _vp]
        L.bfaintb_prefill_tile.restype = _u32
        L.bfaintb_prefill_tile.argtypes = [_u32, _u32]
        L.bfaintb_prefill_tile_cols.restype = _u32
        L.bfaintb_prefill_tile_cols.argtypes = [_u32, _u32]
        L.bfaintb_kernel_name.restype = C.c_char_p
        L.bfaintb_kernel_name.argtypes = [C.c_int, C.c_int, _u32, _u32]
        L.bfaintb_error_string.restype = C.c_char_p
        L.bfaintb_error_string.argtypes = [C.c_int]
        L.bfaintb_version.restype = C.c_int
        L.bfaintb_workspace_status.restype = C.c_int
        L.bfaintb_workspace_status.argtypes = [_vp, _vp]
        L.bfaintb_init.restype = C.c_int
        L.bfaintb_init.argtypes = [_vp]
        L.bfaintb_gemm_static.restype = C.c_int
        L.bfaintb_gemm_static.argtypes = [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, C.c_int, _u32, _vp]
        L.bfaintb_gemm_static_scratch_bytes.restype = C.c_size_t
        L.bfaintb_gemm_static_scratch_bytes.argtypes = []
        L.bfaintb_debug_control.restype = C.c_int
        L.bfaintb_debug_control.argtypes = [_u32, _u32]
        L.bfaintb_gemm_plan.restype = C.c_int
        L.bfaintb_gemm_plan.argtypes = [_u32, _u32, _u32, C.c_int, _u32, C.c_int, C.c_int, _u32, C.POINTER(Plan)]
        L.bfaintb_static_scratch_status.restype = C.c_int
        L.bfaintb_static_scratch_status.argtypes = [_vp]
        L.bfaintb_static_scratch_reset.restype = C.c_int
        L.bfaintb_static_scratch_reset.argtypes = [_vp]
        _lib = L
    return _lib


def error_string(code):
    return lib().bfaintb_error_string(int(code)).decode()


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def _stream_handle(stream):
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def variant(m, n, k, weight_bits=8, group_size=0):
    return lib().bfaintb_gemm_variant(m, n, k, weight_bits, group_size)


def split_k(m, n, k, weight_bits=8, group_size=0):
    return lib().bfaintb_gemm_split_k(m, n, k, weight_bits, group_size)


def prefill_tile(m, n):
    """Rows of the tiles (128 or 256) the PREFILL variant uses for an m x n output."""
    return lib().bfaintb_prefill_tile(m, n)


def prefill_tile_cols(m, n):
    """Columns of those tiles (128, also for the tiles of 256 rows x 128 columns; or 256)."""
    return lib().bfaintb_prefill_tile_cols(m, n)


def kernel_name(m, weight_bits=8, group_size=0, which=AUTO):
    return lib().bfaintb_kernel_name(which, weight_bits, group_size, m).decode()


def workspace_bytes(m, n, k, weight_bits=8, group_size=0, which=AUTO, force_split_k=0):
    return lib().bfaintb_gemm_workspace_bytes_ex(m, n, k, weight_bits, group_size, which, force_split_k)


def workspace_init(workspace, nbytes=None, stream=None):
    if nbytes is None:
        nbytes = workspace.numel() * workspace.element_size()
    rc = lib().bfaintb_workspace_init(_ptr(workspace), nbytes, _stream_handle(stream))
    if rc:
        raise BfaintbError(rc, "bfaintb_workspace_init")


def workspace_status(workspace, stream=None):
    """bfaintb_workspace_status: 0, or a negative BFAINTB_ERR_* (never initialised / a split-K wait gave up)."""
    return lib().bfaintb_workspace_status(_ptr(workspace), _stream_handle(stream))


def init(stream=None):
    """bfaintb_init on the current device (kernel attributes, static scratch); needed only before a first call under capture."""
    rc = lib().bfaintb_init(_stream_handle(stream))
    if rc:
        raise BfaintbError(rc, "bfaintb_init")


def gemm_static(c, a, b, scale, m, n, k, lda=None, ldb=None, ldc=None, weight_bits=8, group_size=0, stream=None, check=True):
    """bfaintb_gemm_static: the GEMM on the library's own per-GPU scratch; allocates nothing."""
    rc = lib().bfaintb_gemm_static(_ptr(c), _ptr(a), _ptr(b), _ptr(scale), m, n, k, k if lda is None else lda,
                                   n if ldb is None else ldb, n if ldc is None else ldc, weight_bits, group_size, _stream_handle(stream))
    if rc and check:
        raise BfaintbError(rc, "bfaintb_gemm_static")
    return rc


DEBUG_SPLIT_WAIT_LIMIT, DEBUG_WITHHOLD_PARTIALS, DEBUG_FORCE_ROW_BLOCK, DEBUG_PLAN_COMPUTE_UNITS = 1, 2, 3, 4
ERR_WORKSPACE, ERR_NOT_INITIALISED, ERR_WORKSPACE_POISONED, ERR_STATIC_SCRATCH = -6, -8, -9, -10


class Plan(C.Structure):
    """bfaintb_plan: what a call would launch."""
    _fields_ = [("variant", C.c_int32), ("kernel", _u32), ("tile_rows", _u32), ("tile_cols", _u32), ("waves", _u32), ("splits", _u32),
                ("k_per_workgroup", _u32), ("workgroups", _u32), ("tail_workgroups", _u32), ("launches", _u32), ("compute_units", _u32),
                ("reserved", _u32), ("workspace_bytes", C.c_uint64)]

    def as_dict(self):
        return {f: getattr(self, f) for f, _ in self._fields_ if f != "reserved"}


KERNEL_DECODE_FAMILY, KERNEL_DECODE_SLAB, KERNEL_TILES_128, KERNEL_TILES_128_LDS, KERNEL_TILES_256X128, KERNEL_TILES_256, KERNEL_TILES_256_LDS = range(1, 8)


def plan(m, n, k, weight_bits=8, group_size=0, packed=False, which=AUTO, force_split_k=0):
    """What gemm (or gemm_prepacked, packed=True) would launch for this shape: a Plan.  Host only."""
    out = Plan()
    rc = lib().bfaintb_gemm_plan(m, n, k, weight_bits, group_size, int(bool(packed)), which, force_split_k, C.byref(out))
    if rc:
        raise BfaintbError(rc, "bfaintb_gemm_plan")
    return out


def debug_control(what, value):
    """Test and tuning hooks.  DEBUG_SPLIT_WAIT_LIMIT and DEBUG_WITHHOLD_PARTIALS are refused unless the process has
    BFAINTB_TEST_HOOKS=1 in its environment."""
    rc = lib().bfaintb_debug_control(what, value)
    if rc:
        raise BfaintbError(rc, "bfaintb_debug_control")


def static_scratch_status(stream=None):
    """bfaintb_workspace_status for the scratch of gemm_static on the current device (synchronises): 0 or
    ERR_WORKSPACE_POISONED (negative codes are returned, HIP errors raise)."""
    rc = lib().bfaintb_static_scratch_status(_stream_handle(stream))
    if rc > 0:
        raise BfaintbError(rc, "bfaintb_static_scratch_status")
    return rc


def static_scratch_reset(stream=None):
    """Puts the scratch of gemm_static on the current device back into its at-rest state (asynchronous on the stream)."""
    rc = lib().bfaintb_static_scratch_reset(_stream_handle(stream))
    if rc:
        raise BfaintbError(rc, "bfaintb_static_scratch_reset")


def _epilogue(bias, residual, ldr, n, activation=ACT_NONE):
    ep = Epilogue()
    ep.bias = _ptr(bias)
    ep.residual = _ptr(residual)
    ep.ldr = (n // 2 if activation == ACT_SILU_GATE else n) if ldr is None else ldr
    ep.activation = activation
    return ep


def gemm(c, a, b, scale, m, n, k, lda=None, ldb=None, ldc=None, weight_bits=8, group_size=0, workspace=None,
         workspace_nbytes=None, stream=None, which=AUTO, force_split_k=0, check=True, bias=None, residual=None, ldr=None,
         activation=ACT_NONE):
    """C = A x dequant(B, scale) through bfaintb_gemm_ex, or (AUTO variant only) + bias through bfaintb_gemm_bias,
    + bias + residual through bfaintb_gemm_fused.  Returns the library's return code (raises on non-zero when ``check``)."""
    lda = k if lda is None else lda
    ldb = n if ldb is None else ldb
    ldc = (n // 2 if activation == ACT_SILU_GATE else n) if ldc is None else ldc
    if workspace_nbytes is None:
        workspace_nbytes = 0 if workspace is None or isinstance(workspace, int) else workspace.numel() * workspace.element_size()
    if residual is not None or activation != ACT_NONE:
        if which != AUTO or force_split_k:
            raise ValueError("bfaintb_gemm_fused takes no forced variant or split factor")
        ep = _epilogue(bias, residual, ldr, n, activation)
        rc = lib().bfaintb_gemm_fused(_ptr(c), _ptr(a), _ptr(b), _ptr(scale), C.byref(ep), m, n, k, lda, ldb, ldc, weight_bits, group_size,
                                      _ptr(workspace), workspace_nbytes, _stream_handle(stream))
    elif bias is not None:
        if which != AUTO or force_split_k:
            raise ValueError("bfaintb_gemm_bias takes no forced variant or split factor")
        rc = lib().bfaintb_gemm_bias(_ptr(c), _ptr(a), _ptr(b), _ptr(scale), _ptr(bias), m, n, k, lda, ldb, ldc, weight_bits,
                                     group_size, _ptr(workspace), workspace_nbytes, _stream_handle(stream))
    else:
        rc = lib().bfaintb_gemm_ex(_ptr(c), _ptr(a), _ptr(b), _ptr(scale), m, n, k, lda, ldb, ldc, weight_bits, group_size,
                                   _ptr(workspace), workspace_nbytes, _stream_handle(stream), which, force_split_k)
    if rc and check:
        raise BfaintbError(rc, "bfaintb_gemm")
    return rc


def gemm_reference(c, a, b, scale_f32, m, n, k, lda=None, ldb=None, ldc=None, workspace=None, workspace_nbytes=None, stream=None,
                   which=AUTO, force_split_k=0, check=True):
    """The reference kernel's arithmetic through bfaintb_gemm_reference[_ex]: fp32 scales [n], 8-bit codes, W and C
    narrowed by truncation.  Workspace as for gemm(..., weight_bits=8, group_size=0)."""
    if workspace_nbytes is None:
        workspace_nbytes = 0 if workspace is None or isinstance(workspace, int) else workspace.numel() * workspace.element_size()
    args = (_ptr(c), _ptr(a), _ptr(b), _ptr(scale_f32), m, n, k, k if lda is None else lda, n if ldb is None else ldb,
            n if ldc is None else ldc, _ptr(workspace), workspace_nbytes, _stream_handle(stream))
    if which != AUTO or force_split_k:
        rc = lib().bfaintb_gemm_reference_ex(*args, which, force_split_k)
    else:
        rc = lib().bfaintb_gemm_reference(*args)
    if rc and check:
        raise BfaintbError(rc, "bfaintb_gemm_reference")
    return rc


def prepack_bytes(n, k, weight_bits=8):
    return lib().bfaintb_prepack_bytes(n, k, weight_bits)


def prepack(packed, b, n, k, ldb=None, weight_bits=8, stream=None, check=True):
    """Row-major B -> the packed operand order (bfaintb_prepack); ``packed`` holds prepack_bytes(n, k, bits) bytes."""
    rc = lib().bfaintb_prepack(_ptr(packed), _ptr(b), n, k, n if ldb is None else ldb, weight_bits, _stream_handle(stream))
    if rc and check:
        raise BfaintbError(rc, "bfaintb_prepack")
    return rc


def prepack_colmajor(packed, b, n, k, ldb=None, weight_bits=8, stream=None, check=True):
    """Column-major B ([n, ldb] codes, k contiguous; 4-bit: two rows per byte) -> the packed order (bfaintb_prepack_colmajor)."""
    rc = lib().bfaintb_prepack_colmajor(_ptr(packed), _ptr(b), n, k, k if ldb is None else ldb, weight_bits, _stream_handle(stream))
    if rc and check:
        raise BfaintbError(rc, "bfaintb_prepack_colmajor")
    return rc


def unpack(b, packed, n, k, ldb=None, weight_bits=8, stream=None, check=True):
    rc = lib().bfaintb_unpack(_ptr(b), _ptr(packed), n, k, n if ldb is None else ldb, weight_bits, _stream_handle(stream))
    if rc and check:
        raise BfaintbError(rc, "bfaintb_unpack")
    return rc


def prepacked_variant(m, n, k, weight_bits=8, group_size=0):
    return lib().bfaintb_gemm_prepacked_variant(m, n, k, weight_bits, group_size)


def prepacked_workspace_bytes(m, n, k, weight_bits=8, group_size=0, which=AUTO):
    return lib().bfaintb_gemm_prepacked_workspace_bytes_ex(m, n, k, weight_bits, group_size, which)


def gemm_prepacked(c, a, packed_b, scale, m, n, k, lda=None, ldc=None, weight_bits=8, group_size=0, bias=None, workspace=None,
                   workspace_nbytes=None, stream=None, which=AUTO, check=True, residual=None, ldr=None, activation=ACT_NONE):
    """C = A x dequant(B, scale) (+ bias) with B in the packed order, through bfaintb_gemm_prepacked_ex; with a residual
    (AUTO variant only) through bfaintb_gemm_prepacked_fused."""
    if workspace_nbytes is None:
        workspace_nbytes = 0 if workspace is None or isinstance(workspace, int) else workspace.numel() * workspace.element_size()
    if residual is not None or activation != ACT_NONE:
        if which != AUTO:
            raise ValueError("bfaintb_gemm_prepacked_fused takes no forced variant")
        ep = _epilogue(bias, residual, ldr, n, activation)
        out_n = n // 2 if activation == ACT_SILU_GATE else n
        rc = lib().bfaintb_gemm_prepacked_fused(_ptr(c), _ptr(a), _ptr(packed_b), _ptr(scale), C.byref(ep), m, n, k,
                                                k if lda is None else lda, out_n if ldc is None else ldc, weight_bits, group_size,
                                                _ptr(workspace), workspace_nbytes, _stream_handle(stream))
        if rc and check:
            raise BfaintbError(rc, "bfaintb_gemm_prepacked_fused")
        return rc
    rc = lib().bfaintb_gemm_prepacked_ex(_ptr(c), _ptr(a), _ptr(packed_b), _ptr(scale), _ptr(bias), m, n, k,
                                         k if lda is None else lda, n if ldc is None else ldc, weight_bits, group_size,
                                         _ptr(workspace), workspace_nbytes, _stream_handle(stream), which)
    if rc and check:
        raise BfaintbError(rc, "bfaintb_gemm_prepacked")
    return rc


def save_packed(path, packed, scale, n, k, weight_bits=8, group_size=0, bias=None):
    """Writes header + packed codes + bf16 scales (+ bf16 bias) in the wire form the header declares."""
    h = PackedHeader()
    rc = lib().bfaintb_packed_header_init(C.byref(h), n, k, weight_bits, group_size, 0 if bias is None else 1)
    if rc:
        raise BfaintbError(rc, "bfaintb_packed_header_init")
    parts = [bytes(h), packed.detach().cpu().contiguous().view(-1).numpy().tobytes(),
             scale.detach().cpu().contiguous().view(-1).view(dtype=_torch().int16).numpy().tobytes()]
    if len(parts[1]) != h.payload_bytes or len(parts[2]) != h.scale_bytes:
        raise ValueError("save_packed: tensor sizes do not match the shape")
    if bias is not None:
        parts.append(bias.detach().cpu().contiguous().view(-1).view(dtype=_torch().int16).numpy().tobytes())
        if len(parts[3]) != 2 * n:
            raise ValueError("save_packed: bias must hold n bf16 values")
    with open(path, "wb") as f:
        for part in parts:
            f.write(part)


def load_packed(path, device="cuda"):
    """Reads a file written by save_packed: (header, packed uint8 tensor, scale bf16 [groups, n], bias bf16 [n] or None)."""
    import numpy as np
    torch = _torch()
    with open(path, "rb") as f:
        raw = f.read()
    if len(raw) < C.sizeof(PackedHeader):
        raise ValueError("load_packed: file shorter than the header")
    h = PackedHeader.from_buffer_copy(raw[:C.sizeof(PackedHeader)])
    rc = lib().bfaintb_packed_header_check(C.byref(h))
    if rc:
        raise BfaintbError(rc, "bfaintb_packed_header_check")
    o0 = h.header_bytes
    o1 = o0 + h.payload_bytes
    o2 = o1 + h.scale_bytes
    o3 = o2 + (2 * h.n if h.has_bias else 0)
    if len(raw) != o3:
        raise ValueError("load_packed: file size does not match the header")
    packed = torch.from_numpy(np.frombuffer(raw, np.uint8, h.payload_bytes, o0).copy()).to(device)
    groups = h.k // h.group_size if h.group_size else 1
    scale = torch.from_numpy(np.frombuffer(raw, np.int16, h.scale_bytes // 2, o1).copy()).view(torch.bfloat16).view(groups, h.n).to(device)
    bias = None
    if h.has_bias:
        bias = torch.from_numpy(np.frombuffer(raw, np.int16, h.n, o2).copy()).view(torch.bfloat16).to(device)
    return h, packed, scale, bias


def _torch():
    import torch
    return torch


def dequant(w, b, scale, n, k, ldb=None, ldw=None, weight_bits=8, group_size=0, stream=None, check=True):
    ldb = n if ldb is None else ldb
    ldw = n if ldw is None else ldw
    rc = lib().bfaintb_dequant(_ptr(w), _ptr(b), _ptr(scale), n, k, ldb, ldw, weight_bits, group_size,
                               _stream_handle(stream))
    if rc and check:
        raise BfaintbError(rc, "bfaintb_dequant")
    return rc


def probe_read(src, nbytes=None, stream=None):
    """Streams a buffer through the GPU and discards it (measurement aid: the fetch-only ceiling)."""
    if nbytes is None:
        nbytes = src.numel() * src.element_size()
    rc = lib().bfaintb_probe_read(_ptr(src), nbytes, None, _stream_handle(stream))
    if rc:
        raise BfaintbError(rc, "bfaintb_probe_read")
