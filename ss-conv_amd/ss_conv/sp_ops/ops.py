"""Shape arithmetic and dtype dispatch in front of the native entry points
(reference: ss_conv/sp_ops/ops.py)."""
import torch

from ss_conv import _ext


def _as_list(v, ndim):
    return list(v) if isinstance(v, (list, tuple)) else [v] * ndim


def get_conv_output_size(input_size, kernel_size, stride, padding, dilation):
    """(in + 2p - d(k-1) - 1) // s + 1 per axis; an axis with kernel -1 collapses to 1
    (reference: ops.py:13-23)."""
    out = []
    for a in range(len(input_size)):
        if kernel_size[a] == -1:
            out.append(1)
        else:
            out.append((input_size[a] + 2 * padding[a] - dilation[a] * (kernel_size[a] - 1) - 1)
                       // stride[a] + 1)
    return out


def get_deconv_output_size(input_size, kernel_size, stride, padding, dilation, output_padding):
    """(in - 1) s - 2p + k + output_padding per axis (reference: ops.py:26-36; the dilation
    does not enter)."""
    out = []
    for a in range(len(input_size)):
        if kernel_size[a] == -1:
            raise ValueError("deconv don't support kernel_size < 0")
        out.append((input_size[a] - 1) * stride[a] - 2 * padding[a] + kernel_size[a]
                   + output_padding[a])
    return out


def get_indice_pairs(indices, batch_size, spatial_shape, ksize=3, stride=1, padding=0, dilation=1,
                     out_padding=0, subm=False, transpose=False, grid=None):
    """Rulebook of one convolution / pooling window (reference: ops.py:39-94).
    Returns (outids, indice_pairs, indice_pair_num).  `grid` is accepted and
    ignored: no dense grid is needed."""
    ndim = indices.shape[1] - 1
    ksize = _as_list(ksize, ndim)
    stride = _as_list(stride, ndim)
    padding = _as_list(padding, ndim)
    dilation = _as_list(dilation, ndim)
    out_padding = _as_list(out_padding, ndim)
    for d, s in zip(dilation, stride):
        assert any([s == 1, d == 1]), "don't support this."
    if subm:
        out_shape = spatial_shape
    elif transpose:
        out_shape = get_deconv_output_size(spatial_shape, ksize, stride, padding, dilation,
                                           out_padding)
    else:
        out_shape = get_conv_output_size(spatial_shape, ksize, stride, padding, dilation)
    if ndim != 3:
        raise NotImplementedError("only 3-d rulebooks are built")
    return _ext.get_indice_pairs_3d(indices, batch_size, list(out_shape), list(spatial_shape),
                                    ksize, stride, padding, dilation, out_padding, int(subm),
                                    int(transpose))


def indice_conv_forward(features, filters, indice_pairs, indice_pair_num, num_activate_out,
                        inverse=False, subm=False):
    if filters.dtype == torch.float32:
        return _ext.indice_conv_fp32(features, filters, indice_pairs, indice_pair_num,
                                     num_activate_out, int(inverse), int(subm))
    if filters.dtype == torch.half:
        return _ext.indice_conv_half(features, filters, indice_pairs, indice_pair_num,
                                     num_activate_out, int(inverse), int(subm))
    raise NotImplementedError("convolution is built for float32 and half filters")


def indice_conv_backward(features, filters, out_bp, indice_pairs, indice_pair_num, inverse=False,
                         subm=False):
    """[input_bp, filters_bp] (reference: sp_ops/ops.py:116-150)."""
    if filters.dtype == torch.float32:
        return _ext.indice_conv_backward_fp32(features, filters, out_bp, indice_pairs,
                                              indice_pair_num, int(inverse), int(subm))
    if filters.dtype == torch.half:
        return _ext.indice_conv_backward_half(features, filters, out_bp, indice_pairs,
                                              indice_pair_num, int(inverse), int(subm))
    raise NotImplementedError("convolution is built for float32 and half filters")


def indice_maxpool_forward(features, indice_pairs, indice_pair_num, num_activate_out):
    if features.dtype == torch.float32:
        return _ext.indice_maxpool_fp32(features, indice_pairs, indice_pair_num, num_activate_out)
    if features.dtype == torch.half:
        return _ext.indice_maxpool_half(features, indice_pairs, indice_pair_num, num_activate_out)
    raise NotImplementedError("pooling is built for float32 and half features")


def indice_maxpool_backward(features, out_features, out_bp, indice_pairs, indice_pair_num):
    if features.dtype == torch.float32:
        return _ext.indice_maxpool_backward_fp32(features, out_features, out_bp, indice_pairs,
                                                 indice_pair_num)
    if features.dtype == torch.half:
        return _ext.indice_maxpool_backward_half(features, out_features, out_bp, indice_pairs,
                                                 indice_pair_num)
    raise NotImplementedError("pooling is built for float32 and half features")


def indice_avgpool_forward(features, indice_pairs, indice_pair_num, num_activate_out, summaryrf):
    if features.dtype == torch.float32:
        return _ext.indice_avgpool_fp32(features, indice_pairs, indice_pair_num, num_activate_out,
                                        summaryrf)
    if features.dtype == torch.half:
        return _ext.indice_avgpool_half(features, indice_pairs, indice_pair_num, num_activate_out,
                                        summaryrf)
    raise NotImplementedError("pooling is built for float32 and half features")


def indice_avgpool_backward(features, out_features, out_bp, indice_pairs, indice_pair_num,
                            summaryrf):
    if features.dtype == torch.float32:
        return _ext.indice_avgpool_backward_fp32(features, out_features, out_bp, indice_pairs,
                                                 indice_pair_num, summaryrf)
    if features.dtype == torch.half:
        return _ext.indice_avgpool_backward_half(features, out_features, out_bp, indice_pairs,
                                                 indice_pair_num, summaryrf)
    raise NotImplementedError("pooling is built for float32 and half features")
