"""autograd entry points over the native kernels
(reference: ss_conv/sp_ops/functional.py:22-453; same exported names).

Forward and backward passes run the HIP kernels (float32; the convolution also on half)."""
import torch
from torch.autograd import Function

from ss_conv import _ext
from . import ops


class _ConvBase(Function):
    inverse = False
    subm = False

    @classmethod
    def _run(cls, ctx, features, filters, indice_pairs, indice_pair_num, num_activate_out):
        ctx.save_for_backward(indice_pairs, indice_pair_num, features, filters)
        # what the library noted on the pairs tensor it wrote (order promises, cached plans)
        # travels with the context, should the saved tensor come back as another object
        ctx.ssc_meta = getattr(indice_pairs, "_ssc_meta", None)
        return ops.indice_conv_forward(features, filters, indice_pairs, indice_pair_num,
                                       num_activate_out, cls.inverse, cls.subm)

    @classmethod
    def _grad(cls, ctx, grad_output):
        """(reference: functional.py:38-43, 60-65, 82-87)"""
        indice_pairs, indice_pair_num, features, filters = ctx.saved_tensors
        if ctx.ssc_meta is not None and getattr(indice_pairs, "_ssc_meta", None) is None:
            indice_pairs._ssc_meta = ctx.ssc_meta
        input_bp, filters_bp = ops.indice_conv_backward(
            features, filters, grad_output.contiguous(), indice_pairs, indice_pair_num,
            cls.inverse, cls.subm)
        return input_bp, filters_bp, None, None, None


class SparseConvFunction(_ConvBase):
    @staticmethod
    def forward(ctx, features, filters, indice_pairs, indice_pair_num, num_activate_out):
        return SparseConvFunction._run(ctx, features, filters, indice_pairs, indice_pair_num,
                                       num_activate_out)

    @staticmethod
    def backward(ctx, grad_output):
        return SparseConvFunction._grad(ctx, grad_output)


class SparseInverseConvFunction(_ConvBase):
    inverse = True

    @staticmethod
    def forward(ctx, features, filters, indice_pairs, indice_pair_num, num_activate_out):
        return SparseInverseConvFunction._run(ctx, features, filters, indice_pairs,
                                              indice_pair_num, num_activate_out)

    @staticmethod
    def backward(ctx, grad_output):
        return SparseInverseConvFunction._grad(ctx, grad_output)


class SubMConvFunction(_ConvBase):
    subm = True

    @staticmethod
    def forward(ctx, features, filters, indice_pairs, indice_pair_num, num_activate_out):
        return SubMConvFunction._run(ctx, features, filters, indice_pairs, indice_pair_num,
                                     num_activate_out)

    @staticmethod
    def backward(ctx, grad_output):
        return SubMConvFunction._grad(ctx, grad_output)


class SparseConvRulebookFunction(Function):
    """Rulebook and convolution of a layer that has no cached rulebook, as one autograd node:
    forward(features, filters, indices, batch_size, out_shape, ksize, stride, padding,
    dilation, out_padding, subm) -> (out_features, outids or None when subm, pairs, num).
    Same numbers as get_indice_pairs followed by indice_conv / indice_subm_conv; the host's
    wait for the number of outputs sits behind the work that does not depend on it."""

    @staticmethod
    def forward(ctx, features, filters, indices, batch_size, out_shape, ksize, stride, padding,
                dilation, out_padding, subm):
        out, outids, pairs, num = _ext.rulebook_conv(features, filters, indices, batch_size,
                                                     out_shape, ksize, stride, padding, dilation,
                                                     out_padding, subm)
        ctx.save_for_backward(pairs, num, features, filters)
        ctx.ssc_meta = getattr(pairs, "_ssc_meta", None)
        ctx.subm = bool(subm)
        if subm:  # the outputs are the inputs: nothing new to return
            ctx.mark_non_differentiable(pairs, num)
            return out, None, pairs, num
        ctx.mark_non_differentiable(outids, pairs, num)
        return out, outids, pairs, num

    @staticmethod
    def backward(ctx, grad_output, *unused):
        indice_pairs, indice_pair_num, features, filters = ctx.saved_tensors
        if ctx.ssc_meta is not None and getattr(indice_pairs, "_ssc_meta", None) is None:
            indice_pairs._ssc_meta = ctx.ssc_meta
        input_bp, filters_bp = ops.indice_conv_backward(
            features, filters, grad_output.contiguous(), indice_pairs, indice_pair_num, False,
            ctx.subm)
        return (input_bp, filters_bp) + (None,) * 9


class SparseMaxPoolFunction(Function):
    @staticmethod
    def forward(ctx, features, indice_pairs, indice_pair_num, num_activate_out):
        out = ops.indice_maxpool_forward(features, indice_pairs, indice_pair_num, num_activate_out)
        ctx.save_for_backward(indice_pairs, indice_pair_num, features, out)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        indice_pairs, indice_pair_num, features, out = ctx.saved_tensors
        input_bp = ops.indice_maxpool_backward(features, out, grad_output.contiguous(),
                                               indice_pairs, indice_pair_num)
        return input_bp, None, None, None


class SparseAvgPoolFunction(Function):
    """use_gs=True (the only value any caller passes) divides by the kernel
    volume; use_gs=False by the number of contributing inputs
    (reference: functional.py:162-185)."""

    @staticmethod
    def forward(ctx, features, indice_pairs, indice_pair_num, num_activate_out, use_gs=True):
        if use_gs:
            summaryrf = torch.full((int(num_activate_out),), int(indice_pairs.shape[0]),
                                   dtype=torch.int32, device=indice_pairs.device)
        else:
            summaryrf = _ext.indiceSummaryRF(indice_pairs, indice_pair_num, num_activate_out)
        out = ops.indice_avgpool_forward(features, indice_pairs, indice_pair_num,
                                         num_activate_out, summaryrf)
        ctx.save_for_backward(indice_pairs, indice_pair_num, features, out, summaryrf)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        indice_pairs, indice_pair_num, features, out, summaryrf = ctx.saved_tensors
        input_bp = ops.indice_avgpool_backward(features, out, grad_output.contiguous(),
                                               indice_pairs, indice_pair_num, summaryrf)
        return input_bp, None, None, None, None


class _SegmentPool(Function):
    @staticmethod
    def _alloc(feats, proposals_offset):
        n_seg = proposals_offset.size(0) - 1
        c = feats.size(1)
        assert feats.is_contiguous()
        assert proposals_offset.is_contiguous()
        out = torch.zeros((n_seg, c), dtype=torch.float32, device=feats.device)
        idx = torch.zeros((n_seg, c), dtype=torch.int32, device=feats.device)
        return n_seg, c, out, idx


class GlobalMaxPool(Function):
    @staticmethod
    def forward(ctx, feats, proposals_offset):
        """feats [sum_n, C] float32, proposals_offset [B+1] int32 -> [B, C]."""
        n_seg, c, out, idx = _SegmentPool._alloc(feats, proposals_offset)
        _ext.global_maxpool_fp(feats, proposals_offset, out, idx, n_seg, c)
        ctx.for_backwards = (idx, proposals_offset, feats.size(0))
        return out

    @staticmethod
    def backward(ctx, d_output_feats):
        idx, proposals_offset, n_rows = ctx.for_backwards
        n_seg, c = d_output_feats.size()
        d_feats = torch.zeros((n_rows, c), dtype=torch.float32, device=d_output_feats.device)
        _ext.global_maxpool_bp(d_feats, proposals_offset, idx, d_output_feats.contiguous(), n_seg, c)
        return d_feats, None


class GlobalAvgPool(Function):
    @staticmethod
    def forward(ctx, feats, proposals_offset):
        """feats [sum_n, C] float32, proposals_offset [B+1] int32 -> [B, C]."""
        n_seg, c, out, idx = _SegmentPool._alloc(feats, proposals_offset)
        _ext.global_avgpool_fp(feats, proposals_offset, out, idx, n_seg, c)
        ctx.for_backwards = (idx, proposals_offset, feats.size(0))
        return out

    @staticmethod
    def backward(ctx, d_output_feats):
        idx, proposals_offset, n_rows = ctx.for_backwards
        n_seg, c = d_output_feats.size()
        # every row is written by the kernel (zero outside the segments): no zero fill first
        d_feats = torch.empty((n_rows, c), dtype=torch.float32, device=d_output_feats.device)
        _ext.global_avgpool_bp(d_feats, proposals_offset, idx, d_output_feats.contiguous(), n_seg, c)
        return d_feats, None


class Voxelization(Function):
    @staticmethod
    def forward(ctx, feats, map_rule, mode=4):
        """feats [N, C], map_rule [M, maxActive+1] int32 -> [M, C]."""
        assert map_rule.is_contiguous()
        assert feats.is_contiguous()
        n, c = feats.size()
        m = map_rule.size(0)
        max_active = map_rule.size(1) - 1
        out = torch.zeros((m, c), dtype=torch.float32, device=feats.device)
        ctx.for_backwards = (map_rule, mode, max_active, n)
        _ext.voxelize_fp(feats, out, map_rule, mode, m, max_active, c)
        return out

    @staticmethod
    def backward(ctx, d_output_feats):
        map_rule, mode, max_active, n = ctx.for_backwards
        m, c = d_output_feats.size()
        d_feats = torch.zeros((n, c), dtype=torch.float32, device=d_output_feats.device)
        _ext.voxelize_bp(d_output_feats.contiguous(), d_feats, map_rule, mode, m, max_active, c)
        return d_feats, None, None


class Voxel2Point_Map(Function):
    @staticmethod
    def forward(ctx, inverse, nActive, maxActive, mode=4):
        """inverse [N] (voxel of each point) -> int32 [nActive, maxActive+1]:
        column 0 the point count, then the point ids (ascending)."""
        inverse = inverse.view(-1).contiguous().int()
        n = inverse.size(0)
        dev = inverse.device
        ids = torch.arange(n, dtype=torch.int32, device=dev)
        if mode == 3 or mode == 4:
            maps = torch.zeros((nActive, maxActive + 1), dtype=torch.int32, device=dev)
        elif mode == 2:
            maps = torch.full((nActive, maxActive + 1), -1, dtype=torch.int32, device=dev)
        elif mode == 1:
            maps = torch.full((nActive, maxActive + 1), n, dtype=torch.int32, device=dev)
        else:
            assert False
        _ext.voxel2point_map(inverse, ids, maps, n, maxActive, mode)
        return maps

    @staticmethod
    def backward(ctx, grad=None):
        return None, None, None, None


class ThreeNN(Function):
    @staticmethod
    def forward(ctx, unknown, known):
        """unknown [n, 4], known [m, 4] rows of (b, x, y, z) -> (dist [n, 3], idx [n, 3] int32)."""
        assert unknown.is_contiguous()
        assert known.is_contiguous()
        n = unknown.size(0)
        m = known.size(0)
        dist2 = torch.empty((n, 3), dtype=torch.float32, device=unknown.device)
        idx = torch.empty((n, 3), dtype=torch.int32, device=unknown.device)
        _ext.three_nn(n, m, unknown, known, dist2, idx)
        return torch.sqrt(dist2), idx

    @staticmethod
    def backward(ctx, a=None, b=None):
        return None, None


class ThreeInterpolate(Function):
    @staticmethod
    def forward(ctx, features, idx, weight):
        """features [m, C], idx [n, 3] int32, weight [n, 3] -> [n, C]."""
        assert features.is_contiguous()
        assert idx.is_contiguous()
        assert weight.is_contiguous()
        m, c = features.size()
        n = idx.size(0)
        ctx.three_interpolate_for_backward = (idx, weight, m)
        out = torch.empty((n, c), dtype=torch.float32, device=features.device)
        _ext.three_interpolate_fp(c, m, n, features, idx, weight, out)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        idx, weight, m = ctx.three_interpolate_for_backward
        n, c = grad_out.size()
        grad_features = torch.zeros((m, c), dtype=torch.float32, device=grad_out.device)
        _ext.three_interpolate_bp(c, n, m, grad_out.contiguous(), idx, weight, grad_features)
        return grad_features, None, None


indice_conv = SparseConvFunction.apply
indice_inverse_conv = SparseInverseConvFunction.apply
indice_subm_conv = SubMConvFunction.apply
rulebook_conv = SparseConvRulebookFunction.apply
indice_maxpool = SparseMaxPoolFunction.apply
indice_avgpool = SparseAvgPoolFunction.apply
global_maxpool = GlobalMaxPool.apply
global_avgpool = GlobalAvgPool.apply
voxelization = Voxelization.apply
voxel2point_mapping = Voxel2Point_Map.apply
three_nn = ThreeNN.apply
three_interpolate = ThreeInterpolate.apply
