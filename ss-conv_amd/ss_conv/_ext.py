"""Binding of libssc.so (include/ssc.h) under the names of the reference's
pybind module ``ss_conv._ext`` (src/ss_conv_ops_api.cpp:15-55).

torch supplies device memory and the current stream; all work happens in the
HIP kernels of the library.  There is no CPU fallback: without the built
library the import fails, and without a GPU every call raises.
"""
import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libssc.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libssc.so is not built (%s missing): run `python ss-conv_amd/build.py`" % LIB_PATH)

_lib = ctypes.CDLL(LIB_PATH)

_vp = ctypes.c_void_p
_i32 = ctypes.c_int32
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t


class Geometry(ctypes.Structure):
    """struct ssc_geometry."""
    _fields_ = [("batch_size", _i32), ("out_shape", _i32 * 3), ("ksize", _i32 * 3),
                ("stride", _i32 * 3), ("padding", _i32 * 3), ("dilation", _i32 * 3),
                ("subm", _i32), ("transpose", _i32)]


_gp = ctypes.POINTER(Geometry)

_SIGNATURES = {
    "ssc_version": (ctypes.c_int, []),
    "ssc_last_error": (ctypes.c_char_p, []),
    "ssc_rulebook_workspace_bytes": (_sz, [_gp, _i64]),
    "ssc_rulebook_count": (ctypes.c_int, [_vp, _i64, _gp, _vp, _sz, ctypes.POINTER(_i32), _vp]),
    "ssc_rulebook_count_ordered": (ctypes.c_int, [_vp, _i64, _gp, _vp, _sz, ctypes.POINTER(_i32),
                                                  ctypes.POINTER(_i32), _vp]),
    "ssc_rulebook_emit": (ctypes.c_int, [_vp, _i64, _gp, _vp, _sz, _vp, _vp, _vp, _vp]),
    "ssc_rulebook_out_bound": (_sz, [_gp, _i64]),
    "ssc_rulebook_clean_table_bytes": (_sz, [_gp, _i64]),
    "ssc_rulebook_begin": (ctypes.c_int, [_vp, _i64, _gp, _vp, _sz, _vp, _vp, _vp, _i64, _vp, _sz,
                                          _vp]),
    "ssc_rulebook_finish": (ctypes.c_int, [_gp, _i64, ctypes.POINTER(_i32), ctypes.POINTER(_i32)]),
    "ssc_rulebook_rows": (ctypes.c_int, [_gp, _i64, _vp, _sz, _vp, _vp]),
    "ssc_rulebook_conv_begin": (ctypes.c_int, [_vp, _i64, _gp, _vp, _sz, _vp, _vp, _vp, _i64, _vp,
                                               _sz, _i32, _i32, _i32, _vp, _sz, _vp, _vp]),
    "ssc_rulebook_conv_finish": (ctypes.c_int, [_gp, _i64, ctypes.POINTER(_i32),
                                                ctypes.POINTER(_i32), _vp, _vp, _i32, _i32, _i32,
                                                _vp, _sz, _vp, _sz, _vp]),
    "ssc_conv_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32, _i64]),
    "ssc_conv_plan_bytes": (_sz, [_i64, _i32, _i32, _i32, _i64]),
    "ssc_conv_plan_scratch_bytes": (_sz, [_i64, _i32, _i32, _i32, _i64]),
    "ssc_conv_packed_bytes": (_sz, [_i32, _i32, _i32]),
    "ssc_conv_tile_cut": (ctypes.c_int, [_i32, _i32, _i32, ctypes.POINTER(_i32),
                                         ctypes.POINTER(_i32), ctypes.POINTER(_i32)]),
    "ssc_conv_plan_build": (ctypes.c_int, [_vp, _i64, _vp, _i32, _i32, _i32, _i64, _i64, _i32, _i32,
                                           _i32, _vp, _sz, _vp, _sz, _vp]),
    "ssc_conv_pack_filters_f32": (ctypes.c_int, [_vp, _i64, _i64, _i64, _i32, _i32, _i32, _vp, _sz,
                                                 _vp]),
    "ssc_conv_pack_filters_f16": (ctypes.c_int, [_vp, _i64, _i64, _i64, _i32, _i32, _i32, _vp, _sz,
                                                 _vp]),
    "ssc_conv_run_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _sz, _vp, _sz, _i64, _i32, _i32, _vp,
                                        _i64, _vp]),
    "ssc_conv_run_f16": (ctypes.c_int, [_vp, _i64, _i32, _vp, _sz, _vp, _sz, _i64, _i32, _i32, _vp,
                                        _i64, _vp]),
    "ssc_conv_run_epilogue_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _sz, _vp, _sz, _i64, _i32,
                                                 _i32, _vp, _vp, _i64, _vp]),
    "ssc_conv_run_epilogue_f16": (ctypes.c_int, [_vp, _i64, _i32, _vp, _sz, _vp, _sz, _i64, _i32,
                                                 _i32, _vp, _vp, _i64, _vp]),
    "ssc_conv_fwd_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _i64, _i64, _i32, _vp, _i64,
                                        _vp, _i32, _i32, _i32, _vp, _i64, _vp, _sz, _vp]),
    "ssc_conv_fwd_f16": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _i64, _i64, _i32, _vp, _i64,
                                        _vp, _i32, _i32, _i32, _vp, _i64, _vp, _sz, _vp]),
    "ssc_conv_bwd_filter_workspace_bytes": (_sz, [_i32, _i32, _i32, _i64]),
    "ssc_conv_bwd_filter_f16": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _i32, _vp, _i64, _vp,
                                               _i32, _i32, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "ssc_conv_bwd_filter_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i64, _i32, _vp, _i64, _vp,
                                               _i32, _i32, _vp, _i64, _i64, _i64, _vp, _sz, _vp]),
    "ssc_pool_max_bwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64,
                                            _vp, _sz, _vp]),
    "ssc_pool_avg_bwd_f32": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _vp, _i64, _vp,
                                            _sz, _vp]),
    "ssc_pool_max_bwd_f16": (ctypes.c_int, [_vp, _vp, _vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64,
                                            _vp, _sz, _vp]),
    "ssc_pool_avg_bwd_f16": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _vp, _i64, _vp,
                                            _sz, _vp]),
    "ssc_segment_avg_bwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "ssc_segment_max_bwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32, _i32, _vp]),
    "ssc_voxel_reduce_bwd_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _vp]),
    "ssc_three_interp_bwd_f32": (ctypes.c_int, [_i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "ssc_profile_conv": (ctypes.c_int, [_i32]),
    "ssc_index_beside_conv": (ctypes.c_int, [_i32]),
    "ssc_conv_tuning": (ctypes.c_int, [_i32]),
    "ssc_profile_conv_read": (ctypes.c_int, [ctypes.POINTER(ctypes.c_float), _i32,
                                             ctypes.POINTER(_i32)]),
    "ssc_kernel_combine_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32,
                                              _vp, _vp]),
    "ssc_kernel_combine_packed_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32,
                                                     _i32, _vp, _vp, _sz, _vp]),
    "ssc_pool_workspace_bytes": (_sz, [_i64, _i32]),
    "ssc_pool_max_f32": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64, _vp, _sz,
                                        _vp]),
    "ssc_pool_max_static_f32": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64, _vp]),
    "ssc_pool_avg_f32": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _vp, _i64, _vp,
                                        _sz, _vp]),
    "ssc_pool_max_f16": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64, _vp, _sz,
                                        _vp]),
    "ssc_pool_max_static_f32": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _i64, _vp]),
    "ssc_pool_avg_f16": (ctypes.c_int, [_vp, _i32, _vp, _i64, _vp, _i32, _vp, _vp, _i64, _vp,
                                        _sz, _vp]),
    "ssc_summary_rf": (ctypes.c_int, [_vp, _i64, _vp, _i32, _vp, _i64, _vp, _sz, _vp]),
    "ssc_segment_avg_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i32, _vp]),
    "ssc_segment_max_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "ssc_voxel_coords": (ctypes.c_int, [_vp, _vp, _i64, ctypes.POINTER(ctypes.c_float),
                                        ctypes.POINTER(ctypes.c_float), _vp, _vp]),
    "ssc_p2v_workspace_bytes": (_sz, [_i64]),
    "ssc_p2v_scan": (ctypes.c_int, [_vp, _vp, _i64, ctypes.POINTER(ctypes.c_float), _vp, _sz,
                                    _vp, _vp, _vp, _vp]),
    "ssc_p2v_compact": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32, ctypes.POINTER(ctypes.c_float),
                                       ctypes.POINTER(ctypes.c_float), _vp, _sz, _vp, _vp, _vp,
                                       _vp, _vp, _vp]),
    "ssc_p2v_voxelize_workspace_bytes": (_sz, [_i64, _i32, ctypes.POINTER(_i32)]),
    "ssc_p2v_voxelize_f32": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i32,
                                            ctypes.POINTER(ctypes.c_float),
                                            ctypes.POINTER(ctypes.c_float), ctypes.POINTER(_i32),
                                            _i32, _i32, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                            _vp, _vp, _vp, _vp, _vp]),
    "ssc_p2v_voxelize_bwd_f32": (ctypes.c_int, [_vp, _i32, _vp, _vp, _vp, _vp, _i32, _i64, _vp,
                                                _vp]),
    "ssc_unique_workspace_bytes": (_sz, [ctypes.POINTER(_i32), _i64]),
    "ssc_unique_build": (ctypes.c_int, [_vp, _i64, ctypes.POINTER(_i32), _vp, _sz, _vp, _vp,
                                        ctypes.POINTER(_i32), _vp]),
    "ssc_unique_rows": (ctypes.c_int, [ctypes.POINTER(_i32), _i64, _vp, _sz, _vp, _vp]),
    "ssc_unique_count": (ctypes.c_int, [_vp, _i64, ctypes.POINTER(_i32), _vp, _sz,
                                        ctypes.POINTER(_i32), _vp]),
    "ssc_unique_emit": (ctypes.c_int, [_vp, _i64, ctypes.POINTER(_i32), _vp, _sz, _i64, _vp, _vp,
                                       _vp, _vp]),
    "ssc_voxel_map": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp]),
    "ssc_voxel_reduce_f32": (ctypes.c_int, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp]),
    "ssc_three_nn": (ctypes.c_int, [_i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "ssc_three_nn_workspace_bytes": (_sz, [_i32]),
    "ssc_three_nn_ws": (ctypes.c_int, [_i32, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ssc_three_nn_grid_workspace_bytes": (_sz, [_i32, _i32, _i32, ctypes.POINTER(_i32)]),
    "ssc_three_nn_grid": (ctypes.c_int, [_i32, _i32, _vp, _vp, _vp, _i32, ctypes.POINTER(_i32),
                                         ctypes.POINTER(ctypes.c_float),
                                         ctypes.POINTER(ctypes.c_float), _vp, _vp, _vp, _sz, _vp]),
    "ssc_three_interp_f32": (ctypes.c_int, [_i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "ssc_v2p_workspace_bytes": (_sz, [_i32, _i32, _i32, ctypes.POINTER(_i32)]),
    "ssc_v2p_interpolate_f32": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, _i32, _i32, _i32,
                                               ctypes.POINTER(_i32), ctypes.POINTER(ctypes.c_float),
                                               ctypes.POINTER(ctypes.c_float), _vp, _vp, _vp, _vp,
                                               _sz, _vp]),
    "ssc_bn_workspace_bytes": (_sz, [_i64, _i32]),
    "ssc_bn_prepare_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _vp, _vp, _vp, _i32, _i32,
                                          ctypes.c_float, ctypes.c_float, _vp, _vp, _vp, _vp, _vp,
                                          _vp, _vp, _vp, _vp, _sz, _vp]),
    "ssc_bnact_fwd_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32,
                                         _vp, _i32, _vp]),
    "ssc_bnact_bwd_sums_f32": (ctypes.c_int, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp,
                                              _vp, _vp, _vp, _i32, _i32, _vp, _vp, _sz, _vp]),
    "ssc_field_scale_f32": (ctypes.c_int, [_vp, _i64, _i32, _vp, _i32, _vp, _vp, _vp]),
    "ssc_bnact_bwd_f32": (ctypes.c_int, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp,
                                         _vp, _vp, _i32, _i32, _vp, _vp, _vp, _vp]),
}

for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(_lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

# ssc_conv_tuning changes what plans look like (ranges, column blocks, launches), and a plan
# built under one setting must not be run under another: the kernel would walk a schedule
# that is laid out otherwise.  Every call through this module's handle of the library is
# noted here, and the plans kept with a rulebook are keyed by the setting they were built
# under (_plan_of), so a change leaves the old plans unused instead of misread.
_tuning_now = [1]
_raw_conv_tuning = _lib.ssc_conv_tuning


def _conv_tuning(flags):
    _tuning_now[0] = int(flags)
    return _raw_conv_tuning(int(flags))


_lib.ssc_conv_tuning = _conv_tuning

SSC_EINVAL, SSC_ERUNTIME, SSC_EWORKSPACE, SSC_EHIP = -1, -2, -3, -4


def _check(rc):
    """Map a status code to the exception class the reference raises
    (utils/tensorview.h:70-90: runtime_error -> RuntimeError, invalid_argument -> ValueError)."""
    if rc == 0:
        return
    msg = _lib.ssc_last_error().decode(errors="replace")
    if rc == SSC_EINVAL:
        raise ValueError(msg)
    raise RuntimeError(msg)


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "ss_conv runs on the GPU only: got a tensor on %s (there is no CPU path)" % t.device)


def _ptr(t):
    return t.data_ptr() if t is not None and t.numel() > 0 else None


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _geometry(batch_size, out_shape, ksize, stride, padding, dilation, subm, transpose):
    g = Geometry()
    g.batch_size = int(batch_size)
    for name, val in (("out_shape", out_shape), ("ksize", ksize), ("stride", stride),
                      ("padding", padding), ("dilation", dilation)):
        setattr(g, name, (_i32 * 3)(*[int(v) for v in val]))
    g.subm = int(bool(subm))
    g.transpose = int(bool(transpose))
    return g


# Output rows are written before their number is known when a buffer for the largest
# possible number of them is at most this large; the result is a slice of that buffer.
_ROWS_AHEAD_BYTES = 256 << 20
_ROWS_KEEP_BYTES = 64 << 20  # unused rows of such a buffer beyond which the result is copied out of it
# largest plan / plan scratch allocated for the bound on the number of outputs, before the
# real number has arrived (the scratch is dropped when the plan is built; the plan, kept
# with the rulebook, is at most this much larger than one sized for the real number)
_PLAN_AHEAD_BYTES = 128 << 20


class RulebookMeta(object):
    """What the library knows about a rulebook it wrote itself: for which direction the pairs
    of every offset ascend in the rows that are accumulated into (`canonical`: (forward,
    inverse)), and the convolution plans built over it so far (`plans`, least recently used
    first; at most MAX_PLANS are kept).

    The owner is the SparseTensor: ``plan_dict[indice_key]`` holds it beside
    ``indice_dict[indice_key]`` and travels with it to the layer's outputs.  For the native
    calls, which get tensors and nothing else, a binding to the pairs tensor rides on the
    tensor object (``_ssc_meta``), valid while that tensor's version counter stands where it
    stood: an in-place edit of the pairs makes the convolution treat them as pairs of unknown
    origin.  A pairs tensor of other identity (a clone, a tensor that came back from a
    checkpoint) is bound to the same plans by adopt_meta once it has been compared with the
    tensor the plans were built over."""
    __slots__ = ("version", "canonical", "plans", "pairs_ref")
    MAX_PLANS = 8

    def __init__(self, version, canonical, plans=None, pairs_ref=None):
        import collections
        self.version = version
        self.canonical = canonical
        self.plans = collections.OrderedDict() if plans is None else plans
        self.pairs_ref = pairs_ref  # the tensor the plans were built over

    def get_plan(self, key):
        plan = self.plans.get(key)
        if plan is not None:
            self.plans.move_to_end(key)
        return plan

    def put_plan(self, key, plan):
        self.plans[key] = plan
        self.plans.move_to_end(key)
        while len(self.plans) > RulebookMeta.MAX_PLANS:
            self.plans.popitem(last=False)  # the least recently used one


def rulebook_meta(indice_pairs):
    """The RulebookMeta of a pairs tensor, or None when it has none that still holds."""
    meta = getattr(indice_pairs, "_ssc_meta", None)
    if meta is None or meta.version != indice_pairs._version or \
            indice_pairs.dtype != torch.int32 or not indice_pairs.is_contiguous():
        return None
    return meta


def adopt_meta(indice_pairs, meta):
    """Bind `indice_pairs` to the plans of `meta` (the record a SparseTensor keeps under the
    rulebook's indice_key) when the tensor carries no valid binding of its own: at once when
    it is the tensor the plans were built over, after one comparison of the contents when it
    is another tensor of the same shape (a clone).  Returns the binding in force, or None."""
    own = rulebook_meta(indice_pairs)
    if own is not None or meta is None:
        return own
    ref = meta.pairs_ref
    if ref is None or not indice_pairs.is_cuda or indice_pairs.dtype != torch.int32 or \
            not indice_pairs.is_contiguous() or indice_pairs.shape != ref.shape or \
            indice_pairs.device != ref.device:
        return None
    same = indice_pairs.data_ptr() == ref.data_ptr() and indice_pairs._version == meta.version
    if not same:
        if ref._version != meta.version or not bool(torch.equal(indice_pairs, ref)):
            return None
    bound = RulebookMeta(indice_pairs._version, meta.canonical, plans=meta.plans,
                         pairs_ref=indice_pairs)
    indice_pairs._ssc_meta = bound
    return bound


def forget_packed(filters):
    """Drop the packed copy of `filters` that the convolution keeps with the tensor.  The
    copy is reused while the tensor's version counter stands still, and an edit through
    ``.data`` (``w.data.copy_(...)``, an EMA swap, ``w.data.normal_()``) does not move that
    counter: call this after such an edit."""
    if hasattr(filters, "_ssc_packed"):
        del filters._ssc_packed


# One buffer per (device, stream) that every rulebook call finds all zero and leaves all
# zero (ssc_rulebook_begin's clean_table): zeroed when it is made, grown when a call asks for
# more, dropped when a call fails.
_clean_tables = {}


def _clean_table(nbytes, dev, stream):
    key = (dev.index, stream)
    held = _clean_tables.get(key)
    if held is None or held.numel() < nbytes:
        held = torch.zeros(max(int(nbytes), 1 << 20), dtype=torch.uint8, device=dev)
        _clean_tables[key] = held
    return held


# ---- index work on a stream of its own -------------------------------------------------------
# A rulebook and the plan of the convolution over it depend on the voxel indices only, not on
# the features: they are queued on a second stream of the device (default priority), and the
# kernel that needs them waits for that stream's event on the caller's stream.  A layer's
# rulebook reads the output indices of the rulebook before it -- written on the same second
# stream -- so in a stack of layers the index work of layer i + 1 runs while the convolution
# of layer i still does, and the host, which waits for that stream only, is not held up by
# the convolutions either.  Tensors written there are allocated there (the caching allocator
# reuses a block in the order of the stream it was allocated on) and recorded on the caller's
# stream before they are handed out.
_index_streams = {}  # device index -> _IndexStream
_index_overlap = os.environ.get("SSC_INDEX_STREAM", "1") != "0"
_beside_now = threading.local()  # .on: what the library was last told on this host thread


def _beside(on):
    """Tell the library whether the index work queued next runs on the second stream (it
    then picks kernels that fit beside a convolution)."""
    if getattr(_beside_now, "on", False) != on:
        _lib.ssc_index_beside_conv(1 if on else 0)
        _beside_now.on = on


# The second stream pays where the kernel that waits for the index work -- the convolution of
# this layer, and with it, in a stack of like layers, the one the index work runs beside --
# is several times as long as the index work itself: from an estimated 20 GFLOP of convolution
# on (0.25 ms; the benchmark layer has 25, and gains 10 %; a strided layer of 13 GFLOP behind
# thirteen small launches gains nothing), and for rulebooks without a convolution from a
# million row-offset combinations on.
_INDEX_STREAM_MIN_FLOPS = 2e10
_INDEX_STREAM_MIN_WORK = 1 << 20
_INDEX_AHEAD_EVERY = 8  # the host runs at most about three times this many rulebooks ahead


class _IndexStream(object):
    __slots__ = ("stream", "handle", "calls", "events")

    def __init__(self, dev):
        self.stream = torch.cuda.Stream(device=dev)
        self.handle = self.stream.cuda_stream
        self.calls = 0
        self.events = []


def index_stream(enable):
    """Switch the second stream for index work on or off (on by default; the environment
    variable SSC_INDEX_STREAM=0 switches it off from the start).  Returns the old setting."""
    global _index_overlap
    old = _index_overlap
    _index_overlap = bool(enable)
    return old


def _index_stream_for(dev, main):
    """The device's stream for index work, or None when this call's stays on `main`."""
    if not _index_overlap or torch.cuda.is_current_stream_capturing():
        return None
    st = _index_streams.get(dev.index)
    if st is None:
        st = _index_streams[dev.index] = _IndexStream(dev)
    if st.handle == main.cuda_stream:
        return None
    # The host waits for the second stream only, so nothing else stops it from queueing
    # convolutions faster than they run: every few rulebooks an event goes behind the
    # caller's stream, and the host waits for the one before the one before last.
    st.calls += 1
    if st.calls % _INDEX_AHEAD_EVERY == 0:
        ev = torch.cuda.Event()
        ev.record(main)
        st.events.append(ev)
        if len(st.events) > 2:
            st.events.pop(0).synchronize()
    return st


def _side_ready(t):
    """Whether the second stream may read `t` without waiting for the caller's stream: it
    wrote the tensor itself, or has waited for it once and the tensor has not changed since."""
    return getattr(t, "_ssc_side_ready", None) == t._version


def _mark_side_ready(t):
    t._ssc_side_ready = t._version


class _NoStream(object):
    def __enter__(self):
        return None

    def __exit__(self, *a):
        return False


_no_stream = _NoStream()


def _index_ctx(r):
    """Allocate and queue torch work on the rulebook's stream."""
    return torch.cuda.stream(r.side.stream) if r.side is not None else _no_stream


def _index_done(r, *tensors):
    """The caller's stream goes on behind what the second stream has queued so far, and the
    tensors it will use there are recorded on it."""
    if r.side is None:
        return
    r.main.wait_stream(r.side.stream)
    for t in tensors:
        if t is not None:
            t.record_stream(r.main)


_scratch_held = {}  # (thread, device index, stream, use) -> buffer


def _stream_scratch(dev, stream, key, nbytes):
    """A buffer that only the kernels of one call at a time use, all on `stream`: one per
    host thread, device, stream and use, kept and reused (the kernels of two calls on a
    stream run in order), regrown when a call needs more.  Allocated under whatever torch
    stream is current, which callers make the one the kernels run on."""
    k = (threading.get_ident(), dev.index, stream, key)
    held = _scratch_held.get(k)
    if held is None or held.numel() < nbytes:
        held = _workspace(nbytes, dev)
        _scratch_held[k] = held
    return held


class _PendingRulebook(object):
    """A rulebook between ssc_rulebook_begin and ssc_rulebook_finish: everything whose size
    does not depend on the number of outputs is queued, the host has not waited yet."""
    __slots__ = ("indices", "n", "geometry", "ws", "pairs", "num", "out_buf", "subm", "stream",
                 "bound", "plan", "scratch", "conv", "main", "side")


def _rulebook_begin(indices, batch_size, out_spatial_shape, kernel_size, stride, padding, dilation,
                    out_padding, subm, transpose, conv=None):
    """Queue a rulebook.  With `conv` = (c_in, c_out, element bytes) of the convolution that
    will run over it, and buffers for its plan within reason, the plan's buffers are
    allocated here (for the bound on the number of outputs) and the rulebook is asked to
    deal the output rows to the convolution's workgroups on its way
    (ssc_rulebook_conv_begin)."""
    if indices.dim() != 2 or indices.size(1) != 4:
        raise RuntimeError("indices must be [N, 4] (batch, x, y, z)")
    for lst in (kernel_size, out_spatial_shape, stride, padding, out_padding, dilation):
        if len(lst) != 3:
            raise RuntimeError("geometry lists must have 3 entries")
    _need_gpu(indices)
    if indices.dtype != torch.int32:
        indices = indices.int()
    indices = indices.contiguous()
    n = indices.size(0)
    dev = indices.device
    g = _geometry(batch_size, out_spatial_shape, kernel_size, stride, padding, dilation, subm,
                  transpose)
    gref = ctypes.byref(g)
    K = int(kernel_size[0]) * int(kernel_size[1]) * int(kernel_size[2])
    nbytes = _lib.ssc_rulebook_workspace_bytes(gref, n)
    if nbytes == 0:  # geometry rejected: let the first call produce the message
        nbytes = 256
    r = _PendingRulebook()
    r.indices, r.n, r.geometry, r.subm = indices, n, g, bool(subm)
    r.main = torch.cuda.current_stream(dev)
    if conv is None:
        worth = n * K >= _INDEX_STREAM_MIN_WORK
    else:  # pairs ~ rows * offsets / prod(stride), two flops per pair, input and output channel
        pairs = n * K / max(int(stride[0]) * int(stride[1]) * int(stride[2]), 1)
        worth = 2.0 * pairs * conv[0] * conv[1] >= _INDEX_STREAM_MIN_FLOPS
    r.side = _index_stream_for(dev, r.main) if worth else None
    _beside(r.side is not None)
    if r.side is not None:
        if not _side_ready(indices):
            r.side.stream.wait_stream(r.main)
            _mark_side_ready(indices)
        indices.record_stream(r.side.stream)
        r.stream = r.side.handle
    else:
        r.stream = r.main.cuda_stream
    with _index_ctx(r):
        _rulebook_queue(r, gref, K, nbytes, conv)
    return r


def _rulebook_queue(r, gref, K, nbytes, conv):
    """Allocate a rulebook's buffers and queue it (on the current torch stream = r.stream)."""
    indices, n, subm = r.indices, r.n, r.subm
    dev = indices.device
    # (workspace and plan scratch hold nothing between two calls: kept per stream)
    r.ws = _stream_scratch(dev, r.stream, "rulebook", nbytes)
    r.pairs = torch.empty((K, 2, n), dtype=torch.int32, device=dev)
    r.num = torch.empty((K,), dtype=torch.int32, device=dev)
    # Marking, ranking and the pair lists are queued; the host then waits for the number of
    # outputs only, while the pair lists are still being written.  When room for any
    # possible number of output rows is cheap (n * K rows at most), the rows are written in
    # the same launch as the pairs and the result is a slice of that buffer; otherwise by a
    # launch of their own once the number is known.
    r.out_buf = None
    r.bound = n if subm else 0  # most output rows there can be (0: not known)
    if not subm and n > 0:
        bound = _lib.ssc_rulebook_out_bound(gref, n)
        r.bound = max(int(bound), 0)
        if 0 < bound * 16 <= _ROWS_AHEAD_BYTES:
            r.out_buf = torch.empty((bound, 4), dtype=torch.int32, device=dev)
    r.plan = r.scratch = r.conv = None
    if conv is not None and n > 0 and 0 < r.bound <= 8 * n * K:
        c_in, c_out, eb = conv
        plan_bytes = _lib.ssc_conv_plan_bytes(r.bound, K, c_in, c_out, n)
        scratch_bytes = _lib.ssc_conv_plan_scratch_bytes(r.bound, K, c_in, c_out, n)
        if plan_bytes <= _PLAN_AHEAD_BYTES and scratch_bytes <= _PLAN_AHEAD_BYTES:
            r.plan = _workspace(plan_bytes, dev)
            r.scratch = _stream_scratch(dev, r.stream, "plan", scratch_bytes)
            r.conv = (int(c_in), int(c_out), int(eb))
    clean_bytes = _lib.ssc_rulebook_clean_table_bytes(gref, n)
    clean = _clean_table(clean_bytes, dev, r.stream) if clean_bytes > 0 else None
    # (a layer's filter job rides on the rulebook's first launch when that runs on the
    # caller's stream; on the second stream it would have to wait for the weights there)
    job = _take_combine(K, r.conv[0], r.conv[1], dev, r.stream) \
        if r.conv is not None and r.side is None else None
    try:
        if r.conv is not None:
            _check(_lib.ssc_rulebook_conv_begin(
                _ptr(indices), n, gref, r.ws.data_ptr(), r.ws.numel(), _ptr(r.pairs),
                r.num.data_ptr(), _ptr(r.out_buf), 0 if r.out_buf is None else r.out_buf.size(0),
                _ptr(clean), 0 if clean is None else clean.numel(),
                r.conv[0], r.conv[1], r.conv[2], r.scratch.data_ptr(), r.scratch.numel(),
                ctypes.byref(job) if job is not None else None, r.stream))
        else:
            _check(_lib.ssc_rulebook_begin(_ptr(indices), n, gref, r.ws.data_ptr(), r.ws.numel(),
                                           _ptr(r.pairs), r.num.data_ptr(), _ptr(r.out_buf),
                                           0 if r.out_buf is None else r.out_buf.size(0),
                                           _ptr(clean), 0 if clean is None else clean.numel(),
                                           r.stream))
    except Exception:
        _clean_tables.pop((dev.index, r.stream), None)  # it may not be clean any more
        raise


def _rulebook_conv_wait(r):
    """Wait for the number of outputs of a rulebook begun with `conv` and queue the plan of
    the convolution (ssc_rulebook_conv_finish): (n_out, input rows in key order)."""
    n_out = _i32(0)
    in_order = _i32(0)
    _check(_lib.ssc_rulebook_conv_finish(
        ctypes.byref(r.geometry), r.n, ctypes.byref(n_out), ctypes.byref(in_order),
        _ptr(r.pairs), r.num.data_ptr(), r.conv[0], r.conv[1], r.conv[2], r.plan.data_ptr(),
        r.plan.numel(), r.scratch.data_ptr(), r.scratch.numel(), r.stream))
    return n_out.value, bool(in_order.value)


def _rulebook_wait(r):
    """Wait for the number of outputs: (n_out, whether the input rows came in key order)."""
    n_out = _i32(0)
    in_order = _i32(0)
    _check(_lib.ssc_rulebook_finish(ctypes.byref(r.geometry), r.n, ctypes.byref(n_out),
                                    ctypes.byref(in_order)))
    return n_out.value, bool(in_order.value)


def _rulebook_result(r, n_out, in_order):
    """[outids, pairs, num] of a rulebook whose number of outputs has arrived.  What is left
    to queue goes on the rulebook's stream: callers follow with _index_done."""
    with _index_ctx(r):
        if r.subm:
            outids = r.indices
        elif r.out_buf is not None:
            outids = r.out_buf[:n_out]
            if (r.out_buf.size(0) - n_out) * 16 > _ROWS_KEEP_BYTES:
                outids = outids.clone()  # do not keep a large, mostly unused buffer alive
        else:
            # a geometry may leave no output at all (every candidate clipped): the library
            # still wants a valid pointer, so at least one row is allocated and the result is
            # a slice
            out_buf = torch.empty((max(n_out, 1), 4), dtype=torch.int32, device=r.pairs.device)
            outids = out_buf[:n_out]
            _check(_lib.ssc_rulebook_rows(ctypes.byref(r.geometry), r.n, r.ws.data_ptr(),
                                          r.ws.numel(), out_buf.data_ptr(), r.stream))
    # Pairs of an offset always ascend in the input rows, and in the output rows too when
    # the input rows came in key order: the convolution may then skip its order check
    # (the first flag serves a call that accumulates into output rows, the second one
    # with `inverse`, which accumulates into input rows).
    r.pairs._ssc_meta = RulebookMeta(r.pairs._version, (in_order, True), pairs_ref=r.pairs)
    if r.side is not None:
        _mark_side_ready(outids)
    return [outids, r.pairs, r.num]


def _rulebook_finish(r):
    """Wait for the number of outputs; returns [outids, pairs, num]."""
    n_out, in_order = _rulebook_wait(r)
    res = _rulebook_result(r, n_out, in_order)
    _index_done(r, *res)
    return res


def get_indice_pairs_3d(indices, batch_size, out_spatial_shape, spatial_shape, kernel_size, stride,
                        padding, dilation, out_padding, subm, transpose):
    """src/ss_conv_ops.cu:31 / src/conv/indice_conv.h:21-131.
    Returns [outids[N_out,4], indicePairs[K,2,N], indiceNum[K]] (all int32)."""
    return _rulebook_finish(_rulebook_begin(indices, batch_size, out_spatial_shape, kernel_size,
                                            stride, padding, dilation, out_padding, subm,
                                            transpose))


def _filter_strides(filters, c_in, c_out):
    """Element strides (k, ci, co) of a [*kernel, Cin, Cout] tensor seen as [K, Cin, Cout]."""
    if filters.dim() < 3 or filters.size(-2) != c_in:
        raise RuntimeError("filters must be [*kernel_size, Cin, Cout] with Cin = features.size(1)")
    kdims = filters.shape[:-2]
    kstr = filters.stride()[:-2]
    ok = True
    for a in range(len(kdims) - 1):
        if kdims[a] != 1 and kstr[a] != kstr[a + 1] * kdims[a + 1]:
            ok = False
    if not ok:
        filters = filters.contiguous()
        kstr = filters.stride()[:-2]
    return filters, kstr[-1], filters.stride(-2), filters.stride(-1)


_ENTRIES = {
    torch.float32: (_lib.ssc_conv_fwd_f32, _lib.ssc_conv_pack_filters_f32, _lib.ssc_conv_run_f32,
                    _lib.ssc_conv_bwd_filter_f32),
    torch.float16: (_lib.ssc_conv_fwd_f16, _lib.ssc_conv_pack_filters_f16, _lib.ssc_conv_run_f16,
                    _lib.ssc_conv_bwd_filter_f16),
}


def _packed_filters(owner, filters, fs, K, c_in, c_out, stream):
    """The filters in the kernel's fragment order.  The buffers are kept on the tensor the
    caller passed (`owner`), one per way of reading it (forward, or transposed for the input
    gradient), and reused while that tensor's version counter stands still: evaluation-mode
    layers, whose kernel is synthesised once, pack once."""
    flush_combine()
    key = (filters.data_ptr(), tuple(fs), K, c_in, c_out)
    held = getattr(owner, "_ssc_packed", None)
    if held is None or held[0] != owner._version:
        held = (owner._version, {})
        owner._ssc_packed = held
    packed = held[1].get(key)
    if packed is None:
        packed = _workspace(_lib.ssc_conv_packed_bytes(K, c_in, c_out), filters.device)
        _check(_ENTRIES[filters.dtype][1](_ptr(filters), fs[0], fs[1], fs[2], K, c_in, c_out,
                                         packed.data_ptr(), packed.numel(), stream))
        held[1][key] = packed
    return packed


def prepack_filters(filters, c_in, c_out):
    """Queue the packing of `filters` ([*kernel_size, Cin, Cout], float32 or half, on the GPU)
    now and keep the result on the tensor, so that a convolution called with this tensor
    later finds it: a layer that knows its filters before its rulebook packs them while the
    rulebook is still being built.  Returns the packed buffer (None when nothing was done)."""
    if not filters.is_cuda or filters.dtype not in _ENTRIES:
        return None
    owner = filters
    filters, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    K = 1
    for d in filters.shape[:-2]:
        K *= d
    return _packed_filters(owner, filters, (fs_k, fs_ci, fs_co), K, c_in, c_out, _stream(filters))


def _plan_of(meta, pairs, num, K, c_in, c_out, elem_bytes, n_in, n_out, inverse, dev, stream,
             beside=False):
    """The plan of a (direction, channel counts, element type, row counts) combination over
    a rulebook: built on first use, kept with the rulebook afterwards."""
    stride = pairs.size(2)
    key = (bool(inverse), c_in, c_out, elem_bytes, n_in, n_out, _tuning_now[0])
    plan = meta.get_plan(key)
    if plan is None:
        _beside(beside)
        plan = _workspace(_lib.ssc_conv_plan_bytes(n_out, K, c_in, c_out, stride), dev)
        scratch = _workspace(_lib.ssc_conv_plan_scratch_bytes(n_out, K, c_in, c_out, stride), dev)
        flags = 2 if meta.canonical[1 if inverse else 0] else 0
        _check(_lib.ssc_conv_plan_build(_ptr(pairs), stride, num.data_ptr(), K, int(bool(inverse)),
                                        flags, n_in, n_out, c_in, c_out, elem_bytes,
                                        plan.data_ptr(), plan.numel(), scratch.data_ptr(),
                                        scratch.numel(), stream))
        meta.put_plan(key, plan)
    return plan


class _EpilogueStruct(ctypes.Structure):
    """struct ssc_conv_epilogue of include/ssc.h."""
    _fields_ = [("shift", _vp), ("scale", _vp), ("add", _vp), ("pre_bias", _vp), ("mode", _vp),
                ("gate", _vp), ("dest", _vp), ("gate_run", _vp), ("act_scalar", _i32),
                ("act_gate", _i32), ("c_dest", _i32)]


class ConvEpilogue(object):
    """Tables of ssc_conv_run_epilogue_f32, one entry per filter column (device tensors):
    float32 shift, scale, add, pre_bias; int32 mode, gate, dest; gate_run with two int32 per
    block of 64 columns; the activation codes and the number of columns of the rows that
    are stored."""

    def __init__(self, shift, scale, add, pre_bias, mode, gate, dest, gate_run, act_scalar,
                 act_gate, c_dest):
        self.tensors = (shift, scale, add, pre_bias, mode, gate, dest, gate_run)
        n = shift.numel()
        for t, dt in zip(self.tensors, (torch.float32,) * 4 + (torch.int32,) * 4):
            size = 2 * ((n + 63) // 64) if t is gate_run else n
            if not t.is_cuda or t.dtype != dt or t.numel() != size or not t.is_contiguous():
                raise RuntimeError("epilogue tables: contiguous GPU vectors, float32 constants "
                                   "and int32 tables with one entry per filter column, "
                                   "gate_run with two per block of 64 columns")
        self.c_cols = n
        self.c_dest = int(c_dest)
        self.struct = _EpilogueStruct(*[t.data_ptr() for t in self.tensors], int(act_scalar),
                                      int(act_gate), int(c_dest))


def _run_planned(features, n_in, c_in, packed, plan, pair_stride, K, c_out, n_out, s, epilogue):
    """Queue the kernel over packed filters and a plan; with an epilogue the rows stored are
    those of the normalised, gated result."""
    dev = features.device
    if epilogue is None:
        out = torch.empty((n_out, c_out), dtype=features.dtype, device=dev)
        _check(_ENTRIES[features.dtype][2](_ptr(features), n_in, c_in, packed.data_ptr(),
                                           packed.numel(), plan.data_ptr(), plan.numel(),
                                           pair_stride, K, c_out, _ptr(out), n_out, s))
        return out
    if features.dtype not in (torch.float32, torch.float16) or epilogue.c_cols != c_out:
        raise RuntimeError("a convolution epilogue needs float32 or float16 rows and one table "
                           "entry per filter column")
    out = torch.empty((n_out, epilogue.c_dest), dtype=features.dtype, device=dev)
    # (looked up by name at every call: tests count the calls through these attributes)
    entry = (_lib.ssc_conv_run_epilogue_f32 if features.dtype == torch.float32
             else _lib.ssc_conv_run_epilogue_f16)
    _check(entry(_ptr(features), n_in, c_in, packed.data_ptr(), packed.numel(), plan.data_ptr(),
                 plan.numel(), pair_stride, K, c_out, ctypes.byref(epilogue.struct), _ptr(out),
                 n_out, s))
    return out


def _planned_conv(meta, features, owner, filters, fs, pairs, num, K, c_in, c_out, n_out, inverse,
                  epilogue=None):
    """out[n_out, c_out] through a cached plan: the schedule is built on the first call of a
    (direction, channel counts, element type, row counts) combination over this rulebook
    and reused afterwards; later calls launch the filter packing (unless cached as well)
    and the MFMA kernel only."""
    dev = features.device
    s = _stream(features)
    n_in = features.size(0)
    packed = _packed_filters(owner, filters, fs, K, c_in, c_out, s)
    plan = _plan_of(meta, pairs, num, K, c_in, c_out, features.element_size(), n_in, n_out,
                    inverse, dev, s)
    return _run_planned(features, n_in, c_in, packed, plan, pairs.size(2), K, c_out, n_out, s,
                        epilogue)


def rulebook_conv(features, filters, indices, batch_size, out_spatial_shape, kernel_size, stride,
                  padding, dilation, out_padding, subm, epilogue=None):
    """get_indice_pairs_3d followed by indice_conv_fp32 / indice_conv_half over the new
    rulebook, as a layer without a cached rulebook runs them (ss_conv/sp_ops/conv.py:131-150),
    with the host's wait for the number of outputs placed behind everything that does not
    need it: the rulebook is queued, the filters are packed and every argument is checked
    first; after the wait only the plan and the kernel remain to be queued.
    Returns (out_features, outids, pairs, num)."""
    _need_gpu(features, filters, indices)
    dtype = features.dtype
    if dtype not in _ENTRIES or filters.dtype != dtype:
        raise RuntimeError("rulebook_conv needs float32 or half features and filters of one type")
    features = features.contiguous()
    n_in, c_in = features.shape
    c_out = filters.size(-1)
    eb = features.element_size()
    # Between the host's wake-up and the first launch of the plan the GPU has nothing to do:
    # whatever can be prepared is prepared before the wait.  With a bound on the number of
    # outputs at hand (and buffers of that size within reason) that includes the buffers of
    # the plan, which is then queued straight after the wait by the call that waits; tensors
    # and bookkeeping follow when the kernel is on its way.
    r = _rulebook_begin(indices, batch_size, out_spatial_shape, kernel_size, stride, padding,
                        dilation, out_padding, subm, 0, conv=(c_in, c_out, eb))
    owner = filters
    filters, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    K = r.pairs.size(0)
    kvol = 1
    for d in filters.shape[:-2]:
        kvol *= d
    dev = features.device
    s = r.main.cuda_stream  # the convolution's stream (the rulebook may be on another)
    bad = None
    if kvol != K:
        bad = "filters have %d offsets but the rulebook has %d" % (kvol, K)
    elif n_in != r.n:
        bad = "features and indices must have the same number of rows"
    if bad is not None:
        _rulebook_wait(r)  # (the rulebook is queued: end it before raising)
        _index_done(r)
        raise RuntimeError(bad)
    packed = _packed_filters(owner, filters, (fs_k, fs_ci, fs_co), K, c_in, c_out, s)
    if r.conv is None:
        n_out, in_order = _rulebook_wait(r)
        outids, pairs, num = _rulebook_result(r, n_out, in_order)
        with _index_ctx(r):
            plan = _plan_of(pairs._ssc_meta, pairs, num, K, c_in, c_out, eb, n_in, n_out, False,
                            dev, r.stream, beside=r.side is not None)
        _index_done(r, outids, pairs, num, plan)
        out = _run_planned(features, n_in, c_in, packed, plan, n_in, K, c_out, n_out, s, epilogue)
        return out, outids, pairs, num
    n_out, in_order = _rulebook_conv_wait(r)
    if r.side is not None:
        # (the convolution's stream waits for the other one once, behind everything that was
        # queued there)
        outids, pairs, num = _rulebook_result(r, n_out, in_order)
        _index_done(r, outids, pairs, num, r.plan)
        out = _run_planned(features, n_in, c_in, packed, r.plan, n_in, K, c_out, n_out, s,
                           epilogue)
    else:
        out = _run_planned(features, n_in, c_in, packed, r.plan, n_in, K, c_out, n_out, s,
                           epilogue)
        outids, pairs, num = _rulebook_result(r, n_out, in_order)
    if n_out > 0:
        pairs._ssc_meta.put_plan((False, c_in, c_out, eb, n_in, n_out, _tuning_now[0]), r.plan)
    return out, outids, pairs, num


def _conv_any(features, owner, filters, fs, indice_pairs, pairs, num, K, c_in, c_out, n_out,
              inverse, subm):
    """One convolution call: through the rulebook's cached plan when the pairs tensor is one
    this library wrote, through the one-call entry point (order check, schedule and kernel
    every time) for pairs of any other origin."""
    meta = rulebook_meta(indice_pairs)
    if meta is not None and pairs is indice_pairs:
        return _planned_conv(meta, features, owner, filters, fs, pairs, num, K, c_in, c_out, n_out,
                             inverse)
    out = torch.empty((n_out, c_out), dtype=features.dtype, device=features.device)
    ws = _workspace(_lib.ssc_conv_workspace_bytes(n_out, K, c_in, c_out, pairs.size(2)),
                    features.device)
    _beside(False)
    _check(_ENTRIES[features.dtype][0](
        _ptr(features), features.size(0), c_in, _ptr(filters), fs[0], fs[1], fs[2], c_out,
        _ptr(pairs), pairs.size(2), num.data_ptr(), K, int(bool(inverse)), int(bool(subm)),
        _ptr(out), n_out, ws.data_ptr(), ws.numel(), _stream(features)))
    return out


def _indice_conv(dtype, name, features, filters, indice_pairs, indice_num, num_act_out, inverse,
                 subm):
    _need_gpu(features, filters, indice_pairs)
    if features.dtype != dtype or filters.dtype != dtype:
        raise RuntimeError("%s needs %s features and filters" % (name, dtype))
    features = features.contiguous()
    c_in = features.size(1)
    c_out = filters.size(-1)
    owner = filters
    filters, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    pairs = indice_pairs.int().contiguous() if indice_pairs.dtype != torch.int32 \
        else indice_pairs.contiguous()
    num = indice_num.to(device=features.device, dtype=torch.int32).contiguous()
    K = pairs.size(0)
    kvol = 1
    for d in filters.shape[:-2]:
        kvol *= d
    if kvol != K:
        raise RuntimeError("filters have %d offsets but the rulebook has %d" % (kvol, K))
    return _conv_any(features, owner, filters, (fs_k, fs_ci, fs_co), indice_pairs, pairs, num, K,
                     c_in, c_out, int(num_act_out), inverse, subm)


def indice_conv_epilogue_fp32(features, filters, indice_pairs, indice_num, num_act_out, subm,
                              epilogue):
    """indice_conv_fp32 (forward direction) over a rulebook this library wrote, followed by
    the evaluation-mode batch norm and gate of `epilogue` (ConvEpilogue) while the rows are
    written: the block conv -> bn -> activation of Common_utils/ss_conv_modules.py:105-117
    as one kernel.  `filters` carry one column per table entry."""
    _need_gpu(features, filters, indice_pairs)
    meta = rulebook_meta(indice_pairs)
    if meta is None or indice_pairs.dtype != torch.int32 or not indice_pairs.is_contiguous():
        raise RuntimeError("indice_conv_epilogue_fp32 needs a rulebook built by this library")
    features = features.contiguous()
    c_in = features.size(1)
    c_out = filters.size(-1)
    owner = filters
    filters, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    num = indice_num.to(device=features.device, dtype=torch.int32).contiguous()
    K = indice_pairs.size(0)
    return _planned_conv(meta, features, owner, filters, (fs_k, fs_ci, fs_co), indice_pairs, num, K,
                         c_in, c_out, int(num_act_out), False, epilogue)


def indice_conv_fp32(features, filters, indice_pairs, indice_num, num_act_out, inverse, subm):
    """src/conv/indice_conv.h:247-343 (bound at src/ss_conv_ops_api.cpp:21)."""
    return _indice_conv(torch.float32, "indice_conv_fp32", features, filters, indice_pairs,
                        indice_num, num_act_out, inverse, subm)


def indice_conv_half(features, filters, indice_pairs, indice_num, num_act_out, inverse, subm):
    """indiceConv<at::Half> (src/ss_conv_ops.cu:74-78, bound at src/ss_conv_ops_api.cpp:23):
    half-precision tensors, fp32 arithmetic, one rounding per output element."""
    return _indice_conv(torch.float16, "indice_conv_half", features, filters, indice_pairs,
                        indice_num, num_act_out, inverse, subm)


def _indice_conv_backward(dtype, name, features, filters, out_bp, indice_pairs, indice_num,
                          inverse, subm):
    _need_gpu(features, filters, out_bp, indice_pairs)
    if features.dtype != dtype or filters.dtype != dtype or out_bp.dtype != dtype:
        raise RuntimeError("%s needs %s tensors" % (name, dtype))
    features = features.contiguous()
    out_bp = out_bp.contiguous()
    n_in, c_in = features.shape
    n_out, c_out = out_bp.shape
    owner = filters
    filters, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    pairs = indice_pairs.int().contiguous() if indice_pairs.dtype != torch.int32 \
        else indice_pairs.contiguous()
    num = indice_num.to(device=features.device, dtype=torch.int32).contiguous()
    K = pairs.size(0)
    dev = features.device
    s = _stream(features)
    # input gradient: the forward kernel on out_bp, pairs swapped, filters transposed
    input_bp = _conv_any(out_bp, owner, filters, (fs_k, fs_co, fs_ci), indice_pairs, pairs, num, K,
                         c_out, c_in, n_in, not inverse, subm)
    # filter gradient
    filters_bp = torch.empty(tuple(filters.shape), dtype=dtype, device=dev)
    ws2 = _workspace(_lib.ssc_conv_bwd_filter_workspace_bytes(K, c_in, c_out, pairs.size(2)), dev)
    _check(_ENTRIES[dtype][3](_ptr(features), n_in, c_in, _ptr(out_bp), n_out, c_out, _ptr(pairs),
                              pairs.size(2), num.data_ptr(), K, int(inverse), _ptr(filters_bp),
                              c_in * c_out, c_out, 1, ws2.data_ptr(), ws2.numel(), s))
    return [input_bp, filters_bp]


def indice_conv_backward_fp32(features, filters, out_bp, indice_pairs, indice_num, inverse, subm):
    """src/conv/indice_conv.h:344-426 (bound at src/ss_conv_ops_api.cpp:22): returns
    [input_bp like features, filters_bp shaped like filters]."""
    return _indice_conv_backward(torch.float32, "indice_conv_backward_fp32", features, filters,
                                 out_bp, indice_pairs, indice_num, inverse, subm)


def indice_conv_backward_half(features, filters, out_bp, indice_pairs, indice_num, inverse, subm):
    """indiceConvBackward<at::Half> (src/ss_conv_ops.cu:79-83, bound at
    src/ss_conv_ops_api.cpp:24): half-precision tensors, fp32 arithmetic."""
    return _indice_conv_backward(torch.float16, "indice_conv_backward_half", features, filters,
                                 out_bp, indice_pairs, indice_num, inverse, subm)


_POOL_ENTRIES = {
    torch.float32: ("ssc_pool_max_f32", "ssc_pool_avg_f32", "ssc_pool_max_bwd_f32",
                    "ssc_pool_avg_bwd_f32"),
    torch.half: ("ssc_pool_max_f16", "ssc_pool_avg_f16", "ssc_pool_max_bwd_f16",
                 "ssc_pool_avg_bwd_f16"),
}


def _pool_args(features, indice_pairs, indice_num, dtype):
    _need_gpu(features, indice_pairs)
    if features.dtype != dtype:
        raise RuntimeError("rulebook pooling: expected %s features, got %s" % (dtype, features.dtype))
    features = features.contiguous()
    pairs = indice_pairs.int().contiguous() if indice_pairs.dtype != torch.int32 \
        else indice_pairs.contiguous()
    num = indice_num.to(device=features.device, dtype=torch.int32).contiguous()
    return features, pairs, num


def _same_type(features, *others):
    for t in others:
        if t.dtype != features.dtype:
            raise RuntimeError("rulebook pooling: features and gradients must have one type")


def _maxpool(dtype, features, indice_pairs, indice_num, num_act):
    features, pairs, num = _pool_args(features, indice_pairs, indice_num, dtype)
    n_out, c, K = int(num_act), features.size(1), pairs.size(0)
    out = torch.empty((n_out, c), dtype=dtype, device=features.device)
    ws = _workspace(_lib.ssc_pool_workspace_bytes(n_out, K), features.device)
    _check(getattr(_lib, _POOL_ENTRIES[dtype][0])(
        _ptr(features), c, _ptr(pairs), pairs.size(2), num.data_ptr(), K, _ptr(out), n_out,
        ws.data_ptr(), ws.numel(), _stream(features)))
    return out


def _avgpool(dtype, features, indice_pairs, indice_num, num_act, summaryrf):
    features, pairs, num = _pool_args(features, indice_pairs, indice_num, dtype)
    n_out, c, K = int(num_act), features.size(1), pairs.size(0)
    rf = summaryrf.to(device=features.device, dtype=torch.int32).contiguous()
    if rf.numel() != n_out:
        raise RuntimeError("summaryrf must have one entry per output row")
    out = torch.empty((n_out, c), dtype=dtype, device=features.device)
    ws = _workspace(_lib.ssc_pool_workspace_bytes(n_out, K), features.device)
    _check(getattr(_lib, _POOL_ENTRIES[dtype][1])(
        _ptr(features), c, _ptr(pairs), pairs.size(2), num.data_ptr(), K, _ptr(rf), _ptr(out),
        n_out, ws.data_ptr(), ws.numel(), _stream(features)))
    return out


def _maxpool_backward(dtype, features, out_features, out_bp, indice_pairs, indice_num):
    features, pairs, num = _pool_args(features, indice_pairs, indice_num, dtype)
    out_features = out_features.contiguous()
    out_bp = out_bp.contiguous()
    _need_gpu(out_features, out_bp)
    _same_type(features, out_features, out_bp)
    n_in, c = features.shape
    K = pairs.size(0)
    din = torch.empty((n_in, c), dtype=dtype, device=features.device)
    ws = _workspace(_lib.ssc_pool_workspace_bytes(n_in, K), features.device)
    _check(getattr(_lib, _POOL_ENTRIES[dtype][2])(
        _ptr(features), _ptr(out_features), _ptr(out_bp), c, _ptr(pairs), pairs.size(2),
        num.data_ptr(), K, _ptr(din), n_in, ws.data_ptr(), ws.numel(), _stream(features)))
    return din


def _avgpool_backward(dtype, features, out_bp, indice_pairs, indice_num, summaryrf):
    features, pairs, num = _pool_args(features, indice_pairs, indice_num, dtype)
    out_bp = out_bp.contiguous()
    _need_gpu(out_bp, summaryrf)
    _same_type(features, out_bp)
    rf = summaryrf.int().contiguous()
    n_in, c = features.shape
    K = pairs.size(0)
    din = torch.empty((n_in, c), dtype=dtype, device=features.device)
    ws = _workspace(_lib.ssc_pool_workspace_bytes(n_in, K), features.device)
    _check(getattr(_lib, _POOL_ENTRIES[dtype][3])(
        _ptr(out_bp), c, _ptr(pairs), pairs.size(2), num.data_ptr(), K, _ptr(rf), _ptr(din), n_in,
        ws.data_ptr(), ws.numel(), _stream(features)))
    return din


def indice_maxpool_fp32(features, indice_pairs, indice_num, num_act):
    """src/pool/indice_maxpool.h:15-50."""
    return _maxpool(torch.float32, features, indice_pairs, indice_num, num_act)


def indice_maxpool_half(features, indice_pairs, indice_num, num_act):
    """indice_maxpool_half (src/ss_conv_ops_api.cpp:34): src/pool/indice_maxpool.h:15-50 on
    half rows."""
    return _maxpool(torch.half, features, indice_pairs, indice_num, num_act)


def indice_avgpool_fp32(features, indice_pairs, indice_num, num_act, summaryrf):
    """src/pool/indice_avgpool.h:17-52."""
    return _avgpool(torch.float32, features, indice_pairs, indice_num, num_act, summaryrf)


def indice_avgpool_half(features, indice_pairs, indice_num, num_act, summaryrf):
    """indice_avgpool_half (src/ss_conv_ops_api.cpp:29): every operation rounded to half, as
    at::Half's operators do."""
    return _avgpool(torch.half, features, indice_pairs, indice_num, num_act, summaryrf)


def indice_maxpool_backward_fp32(features, out_features, out_bp, indice_pairs, indice_num):
    """src/pool/indice_maxpool.h:52-86: gradient of the pooled rows routed to the inputs
    that equal the maximum."""
    return _maxpool_backward(torch.float32, features, out_features, out_bp, indice_pairs,
                             indice_num)


def indice_maxpool_backward_half(features, out_features, out_bp, indice_pairs, indice_num):
    """indice_maxpool_backward_half (src/ss_conv_ops_api.cpp:35)."""
    return _maxpool_backward(torch.half, features, out_features, out_bp, indice_pairs, indice_num)


def indice_avgpool_backward_fp32(features, out_features, out_bp, indice_pairs, indice_num,
                                 summaryrf):
    """src/pool/indice_avgpool.h:54-90."""
    return _avgpool_backward(torch.float32, features, out_bp, indice_pairs, indice_num, summaryrf)


def indice_avgpool_backward_half(features, out_features, out_bp, indice_pairs, indice_num,
                                 summaryrf):
    """indice_avgpool_backward_half (src/ss_conv_ops_api.cpp:30)."""
    return _avgpool_backward(torch.half, features, out_bp, indice_pairs, indice_num, summaryrf)


def global_avgpool_bp(d_feats, offsets, out_maxidx, d_out, n_proposal, c):
    """src/pool/global_avgpool.cpp global_avgpool_bp wrapper; fills d_feats in place."""
    _seg_args(d_feats, offsets, d_out, n_proposal, c)
    _check(_lib.ssc_segment_avg_bwd_f32(_ptr(d_out), _ptr(offsets), _ptr(d_feats), d_feats.size(0),
                                        int(n_proposal), int(c), _stream(d_feats)))


def global_maxpool_bp(d_feats, offsets, out_maxidx, d_out, n_proposal, c):
    """src/pool/global_maxpool.cpp global_maxpool_bp wrapper; fills d_feats in place."""
    _seg_args(d_feats, offsets, d_out, n_proposal, c)
    _need_gpu(out_maxidx)
    _check(_lib.ssc_segment_max_bwd_f32(_ptr(d_out), _ptr(out_maxidx.int().contiguous()),
                                        _ptr(d_feats), d_feats.size(0), int(n_proposal), int(c),
                                        _stream(d_feats)))


def voxelize_bp(d_out, d_feats, maps, mode, n_voxel, max_active, c):
    """src/voxelize/voxelize.cpp voxelize_bp wrapper; fills d_feats in place."""
    _need_gpu(d_out, d_feats, maps)
    if d_out.dtype != torch.float32 or d_feats.dtype != torch.float32 or maps.dtype != torch.int32:
        raise RuntimeError("voxelize_bp: wrong dtypes")
    for t in (d_out, d_feats, maps):
        if not t.is_contiguous():
            raise RuntimeError("voxelize_bp needs contiguous tensors")
    _check(_lib.ssc_voxel_reduce_bwd_f32(_ptr(d_out), _ptr(d_feats), _ptr(maps), int(mode),
                                         int(n_voxel), int(max_active), int(c), d_feats.size(0),
                                         _stream(d_out)))


def three_interpolate_bp(c, n, m, grad_out, idx, weight, grad_points):
    """src/voxelize/interpolation.cpp three_interpolate_bp wrapper; fills grad_points in place."""
    _need_gpu(grad_out, idx, weight, grad_points)
    if grad_out.dtype != torch.float32 or weight.dtype != torch.float32 or \
            idx.dtype != torch.int32 or grad_points.dtype != torch.float32:
        raise RuntimeError("three_interpolate_bp: wrong dtypes")
    for t in (grad_out, idx, weight, grad_points):
        if not t.is_contiguous():
            raise RuntimeError("three_interpolate_bp needs contiguous tensors")
    _check(_lib.ssc_three_interp_bwd_f32(int(c), int(n), int(m), _ptr(grad_out), _ptr(idx),
                                         _ptr(weight), _ptr(grad_points), _stream(grad_out)))


def indiceSummaryRF(indice_pairs, indice_num, num_act):
    """src/ss_conv_ops.cu:116-145."""
    _need_gpu(indice_pairs)
    pairs = indice_pairs.int().contiguous() if indice_pairs.dtype != torch.int32 \
        else indice_pairs.contiguous()
    num = indice_num.to(device=pairs.device, dtype=torch.int32).contiguous()
    n_out = int(num_act)
    rf = torch.empty((n_out,), dtype=torch.int32, device=pairs.device)
    _check(_lib.ssc_summary_rf(_ptr(pairs), pairs.size(2), num.data_ptr(), pairs.size(0),
                               _ptr(rf), n_out, None, 0, _stream(pairs)))
    return rf


def _seg_args(feats, offsets, out, n_seg, c):
    _need_gpu(feats, offsets, out)
    if feats.dtype != torch.float32 or offsets.dtype != torch.int32:
        raise RuntimeError("segment pooling needs float32 features and int32 offsets")
    if not (feats.is_contiguous() and offsets.is_contiguous() and out.is_contiguous()):
        raise RuntimeError("segment pooling needs contiguous tensors")
    if offsets.numel() != n_seg + 1 or feats.size(1) != c or out.numel() != n_seg * c:
        raise RuntimeError("segment pooling: inconsistent sizes")


def global_avgpool_fp(feats, offsets, out, out_maxidx, n_proposal, c):
    """src/pool/global_avgpool.cpp:13-20; writes `out` in place."""
    _seg_args(feats, offsets, out, n_proposal, c)
    _check(_lib.ssc_segment_avg_f32(_ptr(feats), offsets.data_ptr(), _ptr(out), n_proposal, c,
                                    _stream(feats)))


def global_maxpool_fp(feats, offsets, out, out_maxidx, n_proposal, c):
    """src/pool/global_maxpool.cpp; writes `out` and `out_maxidx` in place."""
    _seg_args(feats, offsets, out, n_proposal, c)
    if out_maxidx.dtype != torch.int32 or not out_maxidx.is_contiguous():
        raise RuntimeError("out_maxidx must be a contiguous int32 tensor")
    _check(_lib.ssc_segment_max_f32(_ptr(feats), offsets.data_ptr(), _ptr(out), _ptr(out_maxidx),
                                    n_proposal, c, _stream(feats)))


def voxel2point_map(inverse, ids, out_maps, n_point, max_active, mode):
    """src/voxelize/voxel2point.cpp:12-18; fills the pre-initialised `out_maps` in place."""
    _need_gpu(inverse, ids, out_maps)
    for t in (inverse, ids, out_maps):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError("voxel2point_map needs contiguous int32 tensors")
    _check(_lib.ssc_voxel_map(_ptr(inverse), _ptr(ids), _ptr(out_maps), int(n_point),
                              out_maps.size(0), int(max_active), int(mode), _stream(inverse)))


def voxelize_fp(feats, out, maps, mode, n_voxel, max_active, c):
    """src/voxelize/voxelize_cuda_kernel.h:18-40; writes `out` in place."""
    _need_gpu(feats, out, maps)
    if feats.dtype != torch.float32 or maps.dtype != torch.int32:
        raise RuntimeError("voxelize_fp needs float32 features and an int32 map")
    if not (feats.is_contiguous() and out.is_contiguous() and maps.is_contiguous()):
        raise RuntimeError("voxelize_fp needs contiguous tensors")
    _check(_lib.ssc_voxel_reduce_f32(_ptr(feats), _ptr(out), _ptr(maps), int(mode), int(n_voxel),
                                     int(max_active), int(c), _stream(feats)))


def three_nn(n, m, unknown, known, dist2, idx):
    """src/voxelize/interpolation.cpp three_nn wrapper; fills dist2 and idx in place."""
    _need_gpu(unknown, known, dist2, idx)
    if unknown.dtype != torch.float32 or known.dtype != torch.float32 or \
            dist2.dtype != torch.float32 or idx.dtype != torch.int32:
        raise RuntimeError("three_nn: wrong dtypes")
    if unknown.size(-1) != 4 or (known.numel() and known.size(-1) != 4):
        raise RuntimeError("three_nn rows are (b, x, y, z)")
    for t in (unknown, known, dist2, idx):
        if not t.is_contiguous():
            raise RuntimeError("three_nn needs contiguous tensors")
    ws = _workspace(_lib.ssc_three_nn_workspace_bytes(int(m)), unknown.device)
    _check(_lib.ssc_three_nn_ws(int(n), int(m), _ptr(unknown), _ptr(known), _ptr(dist2), _ptr(idx),
                                ws.data_ptr(), ws.numel(), _stream(unknown)))


def three_nn_grid(unknown, known, voxel_indices, batch_size, dims, origin, unit):
    """three_nn for known rows that are the centres of the voxels `voxel_indices` (int32
    [m, 4], distinct, inside a grid of `dims` cells per batch element with cell size `unit`
    and lower corner `origin`): same result, found around each query's own cell.
    Returns (dist2 [n, 3] float32, idx [n, 3] int32)."""
    _need_gpu(unknown, known, voxel_indices)
    if unknown.dtype != torch.float32 or known.dtype != torch.float32 or \
            voxel_indices.dtype != torch.int32:
        raise RuntimeError("three_nn_grid: wrong dtypes")
    if not (unknown.is_contiguous() and known.is_contiguous() and voxel_indices.is_contiguous()):
        raise RuntimeError("three_nn_grid: tensors must be contiguous")
    n, m = unknown.size(0), known.size(0)
    if voxel_indices.size(0) != m:
        raise RuntimeError("three_nn_grid: one voxel row per known row")
    d = (_i32 * 3)(*[int(v) for v in dims])
    o = (ctypes.c_float * 3)(*[float(v) for v in origin])
    u = (ctypes.c_float * 3)(*[float(v) for v in unit])
    nbytes = _lib.ssc_three_nn_grid_workspace_bytes(n, m, int(batch_size), d)
    if nbytes == 0:
        raise RuntimeError("three_nn_grid: batch_size * prod(dims) must be positive and below 2^31")
    ws = _workspace(nbytes, unknown.device)
    dist2 = torch.empty((n, 3), dtype=torch.float32, device=unknown.device)
    idx = torch.empty((n, 3), dtype=torch.int32, device=unknown.device)
    _check(_lib.ssc_three_nn_grid(n, m, _ptr(unknown), _ptr(known), _ptr(voxel_indices),
                                  int(batch_size), d, o, u, _ptr(dist2), _ptr(idx), ws.data_ptr(),
                                  ws.numel(), _stream(unknown)))
    return dist2, idx


class _V2pInterpolate(torch.autograd.Function):
    """Voxel features read back at points, one native call; differentiable in the features
    (the gradient is the interpolation's, through the saved indices and weights)."""

    @staticmethod
    def forward(ctx, feats, points, batch_ids, voxel_indices, batch_size, dims, unit, extent):
        n, m, c = points.size(0), feats.size(0), feats.size(1)
        dev = feats.device
        d = (_i32 * 3)(*[int(v) for v in dims])
        u = (ctypes.c_float * 3)(*[float(v) for v in unit])
        e = (ctypes.c_float * 3)(*[float(v) for v in extent])
        nbytes = _lib.ssc_v2p_workspace_bytes(n, m, int(batch_size), d)
        if nbytes == 0:
            raise RuntimeError("v2p_interpolate: batch_size * prod(dims) must be positive and "
                               "below 2^31")
        ws = _workspace(nbytes, dev)
        out = torch.empty((n, c), dtype=torch.float32, device=dev)
        idx = torch.empty((n, 3), dtype=torch.int32, device=dev)
        weight = torch.empty((n, 3), dtype=torch.float32, device=dev)
        _check(_lib.ssc_v2p_interpolate_f32(_ptr(points), _ptr(batch_ids), n, _ptr(voxel_indices),
                                            _ptr(feats), m, c, int(batch_size), d, u, e, _ptr(out),
                                            _ptr(idx), _ptr(weight), ws.data_ptr(), ws.numel(),
                                            _stream(feats)))
        ctx.saved = (idx, weight, m)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        idx, weight, m = ctx.saved
        n, c = grad_out.size()
        grad = torch.zeros((m, c), dtype=torch.float32, device=grad_out.device)
        three_interpolate_bp(c, n, m, grad_out.contiguous(), idx, weight, grad)
        return (grad,) + (None,) * 7


def v2p_interpolate(feats, points, batch_ids, voxel_indices, batch_size, dims, unit, extent):
    """Voxel2Point.forward with points (ss_conv/sp_ops/voxelize.py:131-160) as one call:
    feats [m, C] float32 of the voxels voxel_indices [m, 4] int32 (distinct), read at
    points [n, 3] float32 of the batch elements batch_ids [n] int64, on a grid of `dims`
    cells of size `unit` that spans `extent` around the origin.  Returns [n, C]."""
    _need_gpu(feats, points, batch_ids, voxel_indices)
    if feats.dtype != torch.float32 or points.dtype != torch.float32 or \
            batch_ids.dtype != torch.int64 or voxel_indices.dtype != torch.int32:
        raise RuntimeError("v2p_interpolate: float32 features and points, int64 ids, int32 voxels")
    if voxel_indices.size(0) != feats.size(0) or feats.size(0) < 1 or \
            batch_ids.size(0) != points.size(0):
        raise RuntimeError("v2p_interpolate: one feature row per voxel (at least one), one id per point")
    return _V2pInterpolate.apply(feats.contiguous(), points.contiguous(), batch_ids.contiguous(),
                                 voxel_indices.contiguous(), batch_size, dims, unit, extent)


def three_interpolate_fp(c, m, n, feats, idx, weight, out):
    """src/voxelize/interpolation.cpp three_interpolate wrapper; fills out in place."""
    _need_gpu(feats, idx, weight, out)
    if feats.dtype != torch.float32 or weight.dtype != torch.float32 or idx.dtype != torch.int32:
        raise RuntimeError("three_interpolate_fp: wrong dtypes")
    for t in (feats, idx, weight, out):
        if not t.is_contiguous():
            raise RuntimeError("three_interpolate_fp needs contiguous tensors")
    _check(_lib.ssc_three_interp_f32(int(c), int(m), int(n), _ptr(feats), _ptr(idx), _ptr(weight),
                                     _ptr(out), _stream(feats)))


# ---- entry points without a counterpart in the reference's binding ---------------------
class _CombineJob(ctypes.Structure):
    """ssc_combine_job of include/ssc.h."""
    _fields_ = [("weight", _vp), ("basis", _vp), ("chan_out", _vp), ("chan_in", _vp),
                ("blocks", _vp), ("n_irreps_in", _i32), ("kernel_volume", _i32), ("out", _vp),
                ("packed", _vp), ("packed_bytes", _sz)]


class _DeferredCombine(object):
    """A synthesis-and-packing of filters that kernel_combine(defer=True) has not queued."""
    __slots__ = ("args", "tensors", "packed", "stream", "sizes")


_deferred_tls = threading.local()


def _deferred_jobs():
    """This host thread's deferred jobs (at most one _DeferredCombine)."""
    jobs = getattr(_deferred_tls, "jobs", None)
    if jobs is None:
        jobs = _deferred_tls.jobs = []
    return jobs


def kernel_combine(weight, basis, chan_out, chan_in, blocks, n_irreps_in, kernel_volume, c_in,
                   c_out, packed=False, defer=False):
    """Dense kernel [K, Cin, Cout] from the flat weight vector and the stacked
    basis (ss_conv/utils/kernel.py:267-299 fused with convolution.py:56).  With `packed`
    the same launch also writes the filters in the convolution kernel's packed order:
    returns (dense, packed buffer).
    With `defer` (and `packed`) nothing is queued yet: the next rulebook_conv on this host
    thread's way takes the work into the first launch of its rulebook, and anything else
    that needs the filters (the packed-filter lookups here) or flush_combine() queues it as
    a launch of its own.  The caller must end with flush_combine() before the tensors can
    be read by anything outside this module."""
    _need_gpu(weight, basis, chan_out, chan_in, blocks)
    flush_combine()
    out = torch.empty((kernel_volume, c_in, c_out), dtype=torch.float32, device=weight.device)
    args = (_ptr(weight), _ptr(basis), _ptr(chan_out), _ptr(chan_in), _ptr(blocks),
            int(n_irreps_in), int(kernel_volume), int(c_in), int(c_out), _ptr(out))
    if not packed:
        _check(_lib.ssc_kernel_combine_f32(*args, _stream(weight)))
        return out
    buf = _workspace(_lib.ssc_conv_packed_bytes(int(kernel_volume), int(c_in), int(c_out)),
                     weight.device)
    if defer:
        job = _DeferredCombine()
        job.args, job.packed, job.stream = args, buf, _stream(weight)
        job.tensors = (weight, basis, chan_out, chan_in, blocks, out)
        job.sizes = (int(kernel_volume), int(c_in), int(c_out), weight.device)
        _deferred_jobs().append(job)
        return out, buf
    _check(_lib.ssc_kernel_combine_packed_f32(*args, buf.data_ptr(), buf.numel(), _stream(weight)))
    return out, buf


def flush_combine():
    """Queue what kernel_combine(defer=True) left, if nobody has taken it."""
    jobs = _deferred_jobs()
    while jobs:
        job = jobs.pop()
        _check(_lib.ssc_kernel_combine_packed_f32(*job.args, job.packed.data_ptr(),
                                                  job.packed.numel(), job.stream))


def _take_combine(K, c_in, c_out, dev, stream):
    """The deferred job as an ssc_combine_job for a rulebook of these sizes on this stream
    (None, and the job queued by itself, when it does not fit)."""
    jobs = _deferred_jobs()
    if not jobs:
        return None
    job = jobs[-1]
    if job.sizes != (K, c_in, c_out, dev) or job.stream != stream:
        flush_combine()
        return None
    jobs.pop()
    a = job.args
    st = _CombineJob(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[9], job.packed.data_ptr(),
                     job.packed.numel())
    st._keep = job  # the tensors outlive the call
    return st


def attach_packed(filters, c_in, c_out, packed):
    """Tell the convolution that `packed` holds `filters` ([*kernel_size, Cin, Cout], float32)
    in its packed order, as prepack_filters would have left it."""
    base, fs_k, fs_ci, fs_co = _filter_strides(filters, c_in, c_out)
    K = 1
    for d in base.shape[:-2]:
        K *= d
    filters._ssc_packed = (filters._version,
                           {(base.data_ptr(), (fs_k, fs_ci, fs_co), K, c_in, c_out): packed})


def voxel_coords(points, batch_ids, half_extent, unit):
    """int32 [N,4] (b, vx, vy, vz) with v = (int)((p + half) / unit) in fp32
    (ss_conv/sp_ops/voxelize.py:85-86)."""
    _need_gpu(points, batch_ids)
    points = points.float().contiguous()
    ids = batch_ids.long().contiguous()
    n = points.size(0)
    coords = torch.empty((n, 4), dtype=torch.int32, device=points.device)
    h = (ctypes.c_float * 3)(*[float(v) for v in half_extent])
    u = (ctypes.c_float * 3)(*[float(v) for v in unit])
    _check(_lib.ssc_voxel_coords(_ptr(points), _ptr(ids), n, h, u, _ptr(coords), _stream(points)))
    return coords


P2V_MAX_IDS = 4096


class _P2vFeatures(torch.autograd.Function):
    """The compacted feature rows as a function of the input rows: row dest[i] of the output
    is row i of the input (rows that stand for empty clouds are zeros), so the gradient of
    input row i is row dest[i] of the output's, or zero for a dropped row."""

    @staticmethod
    def forward(ctx, feats, out_f, dest):
        ctx.save_for_backward(dest)
        ctx.n = feats.size(0)
        return out_f.clone()  # (an output must not be one of the inputs)

    @staticmethod
    def backward(ctx, grad_out):
        (dest,) = ctx.saved_tensors
        kept = dest >= 0
        grad_in = grad_out.new_zeros((ctx.n, grad_out.size(1)))
        grad_in[kept] = grad_out[dest[kept].long()]
        return grad_in, None, None


def p2v_filter(points, feats, batch_ids, half_extent, unit):
    """Filter + batch partition of Point2Voxel.forward (ss_conv/sp_ops/voxelize.py:40-83)
    for float32 points/features and int64 batch ids that are non-decreasing and below
    P2V_MAX_IDS.  Returns None when the inputs do not qualify (or no point survives);
    otherwise (valid_points, valid_feats, valid_ids, voxel_coords, origin_ids, instance_flag)
    with origin_ids / instance_flag as host lists."""
    import numpy as np
    if not (points.is_cuda and feats.is_cuda and batch_ids.is_cuda):
        return None
    if points.dtype != torch.float32 or feats.dtype != torch.float32 or \
            batch_ids.dtype != torch.int64 or points.dim() != 2 or points.size(1) != 3:
        return None
    n = points.size(0)
    if n == 0 or feats.size(0) != n or batch_ids.numel() != n:
        return None
    points, feats, batch_ids = points.contiguous(), feats.contiguous(), batch_ids.contiguous()
    dev = points.device
    ws = _workspace(_lib.ssc_p2v_workspace_bytes(n), dev)
    h = (ctypes.c_float * 3)(*[float(v) for v in half_extent])
    u = (ctypes.c_float * 3)(*[float(v) for v in unit])
    hist_all = np.empty(P2V_MAX_IDS, dtype=np.int32)
    hist_valid = np.empty(P2V_MAX_IDS, dtype=np.int32)
    flags = np.empty(2, dtype=np.int32)
    s = _stream(points)
    _check(_lib.ssc_p2v_scan(_ptr(points), _ptr(batch_ids), n, h, ws.data_ptr(), ws.numel(),
                             hist_all.ctypes.data, hist_valid.ctypes.data, flags.ctypes.data, s))
    if flags[0] or flags[1]:
        return None
    present = hist_all > 0
    alive = hist_valid > 0
    n_valid = int(hist_valid.sum())
    if n_valid == 0:
        return None
    origin_ids = np.nonzero(present)[0]
    m = n_valid + int((present & ~alive).sum())
    c = feats.size(1)
    out_p = torch.empty((m, 3), dtype=torch.float32, device=dev)
    out_f = torch.empty((m, c), dtype=torch.float32, device=dev)
    out_i = torch.empty((m,), dtype=torch.int64, device=dev)
    coords = torch.empty((m, 4), dtype=torch.int32, device=dev)
    needs_grad = torch.is_grad_enabled() and feats.requires_grad
    dest = torch.empty((n,), dtype=torch.int32, device=dev) if needs_grad else None
    _check(_lib.ssc_p2v_compact(_ptr(points), _ptr(feats.detach()), _ptr(batch_ids), n, c, h, u,
                                ws.data_ptr(), ws.numel(), _ptr(out_p), _ptr(out_f), _ptr(out_i),
                                _ptr(coords), _ptr(dest), s))
    if needs_grad:  # keep the point features in the autograd graph
        out_f = _P2vFeatures.apply(feats, out_f, dest)
    return out_p, out_f, out_i, coords, origin_ids, alive[origin_ids].astype(np.float32)


class _P2vVoxelFeatures(torch.autograd.Function):
    """The voxel features of p2v_voxelize as a function of the point features: the forward
    result is handed in (computed with everything else by the one native call); the
    gradient of input row i is mult * grad[voxel of its row], or zero for a dropped row."""

    @staticmethod
    def forward(ctx, feats, voxel_feats, dest, inverse, counts, sel, mode):
        ctx.save_for_backward(dest, inverse, counts)
        ctx.sel, ctx.mode, ctx.shape = sel, mode, tuple(feats.shape)
        return voxel_feats.clone()  # (an output must not be one of the inputs)

    @staticmethod
    def backward(ctx, grad_out):
        dest, inverse, counts = ctx.saved_tensors
        n, c = ctx.shape
        grad_out = grad_out.contiguous()
        grad_in = torch.empty((n, c), dtype=torch.float32, device=grad_out.device)
        _check(_lib.ssc_p2v_voxelize_bwd_f32(_ptr(grad_out), c, dest.data_ptr(),
                                             inverse.data_ptr(), counts.data_ptr(),
                                             _ptr(ctx.sel), ctx.mode, n, grad_in.data_ptr(),
                                             _stream(grad_out)))
        return grad_in, None, None, None, None, None, None


class P2vConsts(object):
    """What p2v_voxelize needs of a module's grid, converted once: half extent, unit and limit
    as the arrays the native call takes."""
    __slots__ = ("half", "unit", "limit", "ws_bytes")

    def __init__(self, half_extent, unit, limit):
        self.half = (ctypes.c_float * 3)(*[float(v) for v in half_extent])
        self.unit = (ctypes.c_float * 3)(*[float(v) for v in unit])
        self.limit = (_i32 * 3)(*[int(v) for v in limit])
        self.ws_bytes = {}  # (points, ids) -> workspace size


def _p2v_scratch_of(dev, stream, key, nbytes):
    """A buffer of the one-call Point2Voxel that nothing reads after the call's kernels."""
    return _stream_scratch(dev, stream, "p2v " + key, nbytes)


def p2v_voxelize(points, feats, batch_ids, consts, mode, n_ids):
    """Point2Voxel.forward (ss_conv/sp_ops/voxelize.py:29-99) in one native call with one
    wait of the host, for float32 points / features and int64 batch ids that are
    non-decreasing and lie in [0, n_ids); `consts` is the grid as a P2vConsts.  Returns None
    when the inputs do not qualify (the caller then takes another path; `n_ids` too small
    counts as not qualifying); otherwise (valid_points [m,3], voxel_feats [v,C],
    voxel_indices [v,4], valid_ids [m], ids present, largest id, alive) with `alive` a host
    array of 0/1 floats over the ids present, or None when every one of them kept points."""
    if not (points.is_cuda and feats.is_cuda and batch_ids.is_cuda):
        return None
    if points.dtype != torch.float32 or feats.dtype != torch.float32 or \
            batch_ids.dtype != torch.int64 or points.dim() != 2 or points.size(1) != 3:
        return None
    n = points.size(0)
    if n == 0 or feats.dim() != 2 or feats.size(0) != n or batch_ids.numel() != n:
        return None
    n_ids = int(n_ids)
    nbytes = consts.ws_bytes.get((n, n_ids))
    if nbytes is None:
        nbytes = _lib.ssc_p2v_voxelize_workspace_bytes(n, n_ids, consts.limit) \
            if 1 <= n_ids <= P2V_MAX_IDS else 0
        if len(consts.ws_bytes) < 64:
            consts.ws_bytes[(n, n_ids)] = nbytes
    if nbytes == 0:
        return None
    points, batch_ids = points.contiguous(), batch_ids.contiguous()
    wants_grad = torch.is_grad_enabled() and feats.requires_grad
    src_feats = feats.detach().contiguous() if feats.requires_grad else feats.contiguous()
    dev = points.device
    c = feats.size(1)
    stream = _stream(points)
    ws = _p2v_scratch_of(dev, stream, "ws", nbytes)
    out_p = torch.empty((n, 3), dtype=torch.float32, device=dev)
    out_i = torch.empty((n,), dtype=torch.int64, device=dev)
    vox_idx = torch.empty((n, 4), dtype=torch.int32, device=dev)
    vox_f = torch.empty((n, c), dtype=torch.float32, device=dev)
    # inverse, counts, dest and (modes 1 / 2) sel side by side: the backward pass reads them,
    # a call without one leaves them in a buffer the next call writes over
    if wants_grad:
        aux = torch.empty((4, n), dtype=torch.int32, device=dev)
        a0 = aux.data_ptr()
    else:
        aux = None
        a0 = _p2v_scratch_of(dev, stream, "aux", 16 * n).data_ptr()
    sel = a0 + 12 * n if mode in (1, 2) else None
    hist = (_i32 * (2 * n_ids))()
    totals = (_i32 * 8)()
    _check(_lib.ssc_p2v_voxelize_f32(
        points.data_ptr(), src_feats.data_ptr(), batch_ids.data_ptr(), n, c, consts.half,
        consts.unit, consts.limit, n_ids, int(mode), ws.data_ptr(), ws.numel(),
        out_p.data_ptr(), out_i.data_ptr(), vox_idx.data_ptr(), vox_f.data_ptr(), a0, a0 + 4 * n,
        a0 + 8 * n, sel, hist, ctypes.byref(hist, 4 * n_ids), totals, stream))
    m, v, flags, present, kept, largest = totals[0], totals[1], totals[2], totals[4], \
        totals[5], totals[6]
    if flags or m == 0 or kept == 0:  # (no point survived at all: the reference's special case)
        return None
    alive = None
    if kept != present:
        import numpy as np
        h = np.frombuffer(hist, dtype=np.int32)
        alive = (h[n_ids:][h[:n_ids] > 0] > 0).astype(np.float32)
    vox_f = vox_f[:v]
    if wants_grad:
        vox_f = _P2vVoxelFeatures.apply(feats, vox_f, aux[2], aux[0], aux[1],
                                        aux[3] if mode in (1, 2) else None, int(mode))
    return out_p[:m], vox_f, vox_idx[:v], out_i[:m], present, largest, alive


def unique_rows(coords, dims, return_counts=True):
    """Sorted unique rows of an int32 [N,4] table with inverse and counts: the
    torch.unique(dim=0, return_inverse=True, return_counts=True) of
    ss_conv/sp_ops/voxelize.py:88 for rows inside `dims`."""
    _need_gpu(coords)
    coords = coords.contiguous()
    n = coords.size(0)
    dev = coords.device
    d = (_i32 * 4)(*[int(v) for v in dims])
    nbytes = _lib.ssc_unique_workspace_bytes(d, n)
    if nbytes == 0:
        raise RuntimeError("unique_rows: prod(dims) must be positive and below 2^31")
    ws = _workspace(nbytes, dev)
    m = _i32(0)
    s = _stream(coords)
    _check(_lib.ssc_unique_count(_ptr(coords), n, d, ws.data_ptr(), ws.numel(), ctypes.byref(m), s))
    uniq = torch.empty((m.value, 4), dtype=torch.int32, device=dev)
    inverse = torch.empty((n,), dtype=torch.int32, device=dev)
    counts = torch.empty((m.value,), dtype=torch.int32, device=dev) if return_counts else None
    _check(_lib.ssc_unique_emit(_ptr(coords), n, d, ws.data_ptr(), ws.numel(), m.value, _ptr(uniq),
                                _ptr(inverse), _ptr(counts), s))
    return uniq, inverse, counts


def unique_rows_max(coords, dims):
    """unique_rows with counts, and the largest count as a Python int, with one wait of the
    host for both sizes (ss_conv/sp_ops/voxelize.py:88-93)."""
    _need_gpu(coords)
    coords = coords.contiguous()
    n = coords.size(0)
    dev = coords.device
    d = (_i32 * 4)(*[int(v) for v in dims])
    nbytes = _lib.ssc_unique_workspace_bytes(d, n)
    if nbytes == 0:
        raise RuntimeError("unique_rows: prod(dims) must be positive and below 2^31")
    ws = _workspace(nbytes, dev)
    inverse = torch.empty((n,), dtype=torch.int32, device=dev)
    counts = torch.empty((max(n, 1),), dtype=torch.int32, device=dev)
    totals = (_i32 * 2)(0, 0)
    s = _stream(coords)
    _check(_lib.ssc_unique_build(_ptr(coords), n, d, ws.data_ptr(), ws.numel(), _ptr(inverse),
                                 counts.data_ptr(), totals, s))
    m = int(totals[0])
    uniq = torch.empty((m, 4), dtype=torch.int32, device=dev)
    _check(_lib.ssc_unique_rows(d, n, ws.data_ptr(), ws.numel(), _ptr(uniq), s))
    return uniq, inverse, counts[:m], int(totals[1])


ACT_NONE, ACT_RELU, ACT_SIGMOID, ACT_TANH = 0, 1, 2, 3


def bn_prepare(x, layout, training, eps, momentum, weight, bias, running_mean, running_var):
    """Per-column constants of the SE(3) batch norm (reference: batchnorm.py:73-112).
    `layout` holds the int32 tables field_of, scalar_idx, field_first, field_dim.
    Updates the running statistics in place when training.
    Returns (shift[c], scale[c], add[c], field_rstd[n_fields])."""
    _need_gpu(x)
    n, c = x.size(0), x.size(1)
    dev = x.device
    n_fields = layout["field_first"].numel()
    shift = torch.empty(c, dtype=torch.float32, device=dev)
    scale = torch.empty(c, dtype=torch.float32, device=dev)
    add = torch.empty(c, dtype=torch.float32, device=dev)
    rstd = torch.empty(n_fields, dtype=torch.float32, device=dev)
    ws = _workspace(_lib.ssc_bn_workspace_bytes(n, c), dev)
    _check(_lib.ssc_bn_prepare_f32(
        _ptr(x), n, c, layout["field_of"].data_ptr(), layout["scalar_idx"].data_ptr(),
        layout["field_first"].data_ptr(), layout["field_dim"].data_ptr(), n_fields,
        int(bool(training)), float(eps), float(momentum), _ptr(weight), _ptr(bias),
        _ptr(running_mean), running_var.data_ptr(), shift.data_ptr(), scale.data_ptr(),
        add.data_ptr(), rstd.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x)))
    return shift, scale, add, rstd


def bnact_forward(x, shift, scale, add, pre_bias, out_mode, gate_col, act_scalar, act_gate, c_out):
    """y[n, c_out] = gated activation of the normalised rows (activation.py:55-100)."""
    _need_gpu(x)
    y = torch.empty((x.size(0), c_out), dtype=torch.float32, device=x.device)
    _check(_lib.ssc_bnact_fwd_f32(_ptr(x), x.size(0), x.size(1), _ptr(shift), _ptr(scale),
                                  _ptr(add), _ptr(pre_bias), _ptr(out_mode), _ptr(gate_col),
                                  int(act_scalar), int(act_gate), _ptr(y), c_out, _stream(x)))
    return y


def bnact_backward_sums(x, dy, shift, scale, add, pre_bias, out_mode, gate_col, gated_first,
                        gated_dim, act_scalar, act_gate):
    """sums[2, c_in]: per input column the sum over rows of dz and of dz * (x - shift)."""
    _need_gpu(x, dy)
    n, c_in = x.size(0), x.size(1)
    sums = torch.empty((2, c_in), dtype=torch.float32, device=x.device)
    ws = _workspace(_lib.ssc_bn_workspace_bytes(n, c_in), x.device)
    _check(_lib.ssc_bnact_bwd_sums_f32(
        _ptr(x), _ptr(dy), n, c_in, dy.size(1), _ptr(shift), _ptr(scale), _ptr(add),
        _ptr(pre_bias), _ptr(out_mode), _ptr(gate_col), _ptr(gated_first), _ptr(gated_dim),
        int(act_scalar), int(act_gate), sums.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x)))
    return sums


def bnact_backward(x, dy, shift, scale, add, pre_bias, out_mode, gate_col, gated_first, gated_dim,
                   act_scalar, act_gate, dz_mean, coef):
    """dx = scale * (dz - dz_mean) - coef * (x - shift)."""
    _need_gpu(x, dy)
    dx = torch.empty_like(x)
    _check(_lib.ssc_bnact_bwd_f32(
        _ptr(x), _ptr(dy), x.size(0), x.size(1), dy.size(1), _ptr(shift), _ptr(scale), _ptr(add),
        _ptr(pre_bias), _ptr(out_mode), _ptr(gate_col), _ptr(gated_first), _ptr(gated_dim),
        int(act_scalar), int(act_gate), _ptr(dz_mean), _ptr(coef), _ptr(dx), _stream(x)))
    return dx


def field_scale(x, scale, field_of):
    """y[r, c] = x[r, c] * scale[r, field_of[c]] for float32 x [n, C], scale [n, F] and an
    int32 table field_of [C] (the multiply of ss_conv/dropout.py:44-45)."""
    _need_gpu(x, scale, field_of)
    if x.dtype != torch.float32 or scale.dtype != torch.float32 or field_of.dtype != torch.int32:
        raise RuntimeError("field_scale: wrong dtypes")
    x = x.contiguous()
    scale = scale.contiguous()
    n, c = x.shape
    if scale.size(0) != n or field_of.numel() != c:
        raise RuntimeError("field_scale: shapes do not match")
    y = torch.empty_like(x)
    _check(_lib.ssc_field_scale_f32(_ptr(x), n, c, _ptr(scale), scale.size(1), _ptr(field_of),
                                    _ptr(y), _stream(x)))
    return y


def profile_conv(enable, every=1):
    """Start (clearing earlier samples) or stop timing of the convolution kernel; with
    `every` = n only every n-th launch is timed."""
    _check(_lib.ssc_profile_conv(max(1, int(every)) if enable else 0))


def profile_conv_read():
    """Durations in ms of the convolution kernel launches recorded since
    profile_conv(True), oldest first (waits for them to finish)."""
    buf = (ctypes.c_float * 512)()
    n = _i32(0)
    _check(_lib.ssc_profile_conv_read(buf, 512, ctypes.byref(n)))
    return [float(buf[i]) for i in range(n.value)]
