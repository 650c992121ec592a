"""Point cloud <-> sparse voxel tensor (reference: ss_conv/sp_ops/voxelize.py:18-162)."""
import numpy as np
import torch
import torch.nn as nn

from ss_conv import _ext
from .tensor import SparseTensor
from .functional import voxelization, voxel2point_mapping, three_nn, three_interpolate


class Point2Voxel(nn.Module):
    """Voxelise a batch of point clouds centred on the origin.

    forward(point_cloud [N,3], feature [N,C], batch_ids [N]) returns
    (valid_points, SparseTensor, valid_ids, valid_instance_flag) as the
    reference does (voxelize.py:29-99): points outside the grid are dropped,
    batch elements left without points get one zero point, points are ordered
    by batch id (stable), voxel index = (int)((p + half_extent) / unit) in fp32,
    voxels come out in ascending (b, x, y, z) order and carry the mean (mode 4),
    sum (3), first (1) or last (2) of their points' features.

    The sorted-unique of voxel rows, the per-voxel point lists and the feature
    reduction are native kernels; row filtering and the batch sort are torch ops.
    """

    _n_ids_seen = 64  # see _n_ids_hint

    def __init__(self, voxel_num_limit=[64, 64, 64], unit_voxel_extent=[0.05, 0.05, 0.05],
                 voxelization_mode=4):
        super().__init__()
        self.unit_voxel_extent = torch.tensor(np.asarray(unit_voxel_extent, dtype=np.float64),
                                              dtype=torch.float32)
        self.voxel_num_limit = np.array(voxel_num_limit)
        self.voxelization_mode = voxelization_mode
        # The one-call path sizes its tables for batch ids below this number before it has
        # looked at the ids (the call checks on the device that they fit, and falls back
        # when they do not): 1 + the largest id of the last call, of this module or, for its
        # first call, of any other (64 before any call).
        self._n_ids_hint = Point2Voxel._n_ids_seen
        self._consts = None
        self._grid_consts()  # (converted here, not by the first call)
        self.last_path = None  # which of the three ways the last forward took (diagnostics)

    def _grid_consts(self):
        """(half extent, unit) as float32 arrays, the same for the one-call path
        (_ext.P2vConsts) and the grid shape as int64: made again when the module's extent or
        limit were changed."""
        key = (self.unit_voxel_extent.numpy().tobytes(), self.voxel_num_limit.tobytes())
        held = self._consts
        if held is None or held[0] != key:
            unit = self.unit_voxel_extent.numpy().astype(np.float32)
            limit = self.voxel_num_limit.astype(np.float32)
            half = np.float32(0.5) * (limit * unit)  # fp32 throughout, as on the device
            held = (key, (half, unit, _ext.P2vConsts(half, unit, self.voxel_num_limit),
                          self.voxel_num_limit.astype(np.int64)))
            self._consts = held
        return held[1]

    def forward(self, point_cloud, feature, batch_ids):
        assert len(point_cloud.size()) == 2
        C = feature.size(1)
        device = point_cloud.device

        # Clouds concatenated in batch order with small non-negative ids: filter and
        # partition in native kernels (one host read); anything else takes the
        # reference's sequence of torch operations below.
        # (the native filter keeps the features in the autograd graph when they carry a
        # gradient, as the reference's boolean-mask indexing does)
        # One native call with one wait of the host when the batch ids lie below the number
        # the tables were sized for (the call checks that on the device).
        if self._n_ids_hint is not None and point_cloud.is_cuda:
            one = _ext.p2v_voxelize(point_cloud, feature, batch_ids, self._grid_consts()[2],
                                    self.voxelization_mode, self._n_ids_hint)
            if one is not None:
                valid_point_cloud, voxel_feats, voxel_index, valid_ids, B1, max_id, alive = one
                valid_instance_flag = torch.ones(B1, dtype=torch.float32, device=device) \
                    if alive is None else torch.from_numpy(alive).to(device)
                # (the rows carry the clouds' own ids: with gaps in the ids the tensor's batch
                # size is 1 + the largest one, so that every row lies inside the grid)
                sparse_feat = SparseTensor(voxel_feats, voxel_index, self._grid_consts()[3].copy(),
                                           max(B1, max_id + 1))
                self.last_path = "one call"
                self._n_ids_hint = Point2Voxel._n_ids_seen = max_id + 1
                return valid_point_cloud, sparse_feat, valid_ids, valid_instance_flag
        half, unit = self._grid_consts()[:2]
        fast = _ext.p2v_filter(point_cloud, feature, batch_ids, half, unit) \
            if point_cloud.is_cuda else None
        if fast is not None:
            valid_point_cloud, valid_feature, valid_ids, voxel_index, origin_ids, alive = fast
            B1 = len(origin_ids)
            self._n_ids_hint = int(origin_ids[-1]) + 1
            self.last_path = "native filter"
            # all clouds kept points (the usual case): a fill on the device instead of a
            # synchronous upload
            valid_instance_flag = torch.ones(B1, dtype=torch.float32, device=device) \
                if bool(alive.all()) else torch.from_numpy(alive).to(device)
            return self._voxelize(valid_point_cloud, valid_feature, valid_ids, voxel_index,
                                  int(origin_ids[-1]), valid_instance_flag, B1)

        self.last_path = "torch filter"
        half_t = torch.from_numpy(half).reshape(1, 3).to(device)
        unique_origin_ids = torch.unique(batch_ids)
        B1 = unique_origin_ids.size(0)
        inside = (torch.abs(point_cloud) > half_t).sum(1) == 0
        if inside.sum() == 0:
            valid_instance_flag = torch.zeros(B1, dtype=torch.float32, device=device)
            valid_point_cloud = torch.zeros(B1, 3, dtype=torch.float32, device=device)
            valid_feature = torch.zeros(B1, C, dtype=torch.float32, device=device)
            valid_ids = unique_origin_ids
        else:
            valid_point_cloud = point_cloud[inside].contiguous()
            valid_feature = feature[inside].contiguous()
            valid_ids = batch_ids[inside].contiguous()
            unique_valid_ids = torch.unique(valid_ids)
            B2 = unique_valid_ids.size(0)
            if B1 == B2:
                valid_instance_flag = torch.ones(B1, dtype=torch.float32, device=device)
            else:
                valid_instance_flag = torch.isin(unique_origin_ids, unique_valid_ids).float()
                invalid_ids = unique_origin_ids[valid_instance_flag == 0].contiguous()
                assert len(invalid_ids) == B1 - B2
                pad = B1 - B2
                valid_point_cloud = torch.cat(
                    [valid_point_cloud, torch.zeros(pad, 3, dtype=torch.float32, device=device)], 0)
                valid_feature = torch.cat(
                    [valid_feature, torch.zeros(pad, C, dtype=torch.float32, device=device)], 0)
                valid_ids = torch.cat([valid_ids, invalid_ids], 0)
            order = torch.sort(valid_ids, stable=True)[1]
            valid_point_cloud = valid_point_cloud[order].contiguous()
            valid_feature = valid_feature[order].contiguous()
            valid_ids = valid_ids[order].contiguous()

        lo = int(valid_ids.min().item())
        hi = int(valid_ids.max().item())
        if lo < 0:
            raise ValueError("batch ids must be non-negative")
        voxel_index = _ext.voxel_coords(valid_point_cloud, valid_ids, half, unit)
        return self._voxelize(valid_point_cloud, valid_feature, valid_ids, voxel_index, hi,
                              valid_instance_flag, B1)

    def _voxelize(self, valid_point_cloud, valid_feature, valid_ids, voxel_index, max_id,
                  valid_instance_flag, B1):
        """Unique voxels, per-voxel point lists and feature reduction (voxelize.py:85-99)."""
        # a point exactly on the upper face lands on index == limit, hence the +1
        dims = [max_id + 1] + [int(v) + 1 for v in self.voxel_num_limit]
        occupied_index, inverse, count, largest = _ext.unique_rows_max(voxel_index, dims)
        nActive = occupied_index.size(0)
        if self.voxelization_mode == 1 or self.voxelization_mode == 2:
            maxActive = 1
        else:
            maxActive = largest
        v2p_maps = voxel2point_mapping(inverse, nActive, maxActive, self.voxelization_mode)
        sparse_feat = voxelization(valid_feature.float().contiguous(), v2p_maps.detach(),
                                   self.voxelization_mode)
        sparse_feat = SparseTensor(sparse_feat, occupied_index.detach(),
                                   self.voxel_num_limit.astype(np.int64), max(B1, max_id + 1))
        return valid_point_cloud, sparse_feat, valid_ids, valid_instance_flag


class Voxel2Point(nn.Module):
    """Read voxel features back at points by inverse-distance interpolation over
    the three nearest voxel centres of the same batch element
    (reference: voxelize.py:102-162).  Without points, returns the voxel
    centres, their features and their batch ids."""

    def __init__(self, voxel_extent=None, unit_voxel_extent=None):
        super().__init__()
        assert voxel_extent is not None or unit_voxel_extent is not None
        self.voxel_extent = None if voxel_extent is None else \
            np.asarray(voxel_extent, dtype=np.float64)
        self.unit_voxel_extent = None if unit_voxel_extent is None else \
            np.asarray(unit_voxel_extent, dtype=np.float64)
        self._consts = {}  # (device, grid shape) -> (unit, extent) on the device

    def forward(self, sparse_feat, point_cloud=None, batch_ids=None):
        if point_cloud is not None and self._one_call_ok(sparse_feat, point_cloud, batch_ids):
            # centres, search, weights and interpolation as one native call
            unit, extent = self._unit_extent(sparse_feat)
            return _ext.v2p_interpolate(
                sparse_feat.features, point_cloud, batch_ids, sparse_feat.indices,
                sparse_feat.batch_size,
                # (a point on the upper face of the grid has voxel index == shape,
                # voxelize.py:85-86)
                [int(v) + 1 for v in sparse_feat.spatial_shape], unit, extent)
        vx_points, vx_feats = self._get_vertice_feats(sparse_feat)
        if point_cloud is not None:
            assert batch_ids is not None
            points = torch.cat([batch_ids.float().unsqueeze(1), point_cloud], dim=1)
            return self._get_point_feats(points.contiguous(), vx_points, vx_feats, sparse_feat)
        return vx_points[:, 1:].contiguous(), vx_feats, vx_points[:, 0].contiguous()

    @staticmethod
    def _one_call_ok(sparse_tensor, point_cloud, batch_ids):
        feat, idx = sparse_tensor.features, sparse_tensor.indices
        return (batch_ids is not None and feat.is_cuda and point_cloud.is_cuda and idx.is_cuda
                and batch_ids.is_cuda and feat.dtype == torch.float32 and feat.dim() == 2
                and point_cloud.dtype == torch.float32 and idx.dtype == torch.int32
                and batch_ids.dtype == torch.int64 and feat.size(0) >= 1
                and point_cloud.dim() == 2 and point_cloud.size(1) == 3)

    def _unit_extent(self, sparse_tensor):
        """(unit, extent) of the voxel grid as float32 host arrays: the numbers that
        _get_vertice_feats puts on the device."""
        shape = np.asarray(sparse_tensor.spatial_shape, dtype=np.float64)
        if self.voxel_extent is not None:
            unit, extent = self.voxel_extent / shape, self.voxel_extent
        else:
            unit, extent = self.unit_voxel_extent, self.unit_voxel_extent * shape
        return (np.asarray(unit, dtype=np.float64).astype(np.float32),
                np.asarray(extent, dtype=np.float64).astype(np.float32))

    def _get_vertice_feats(self, sparse_tensor):
        feat = sparse_tensor.features
        device = feat.device
        # the two 3-vectors depend on the grid shape only: uploaded once (an upload from
        # pageable memory is a synchronous copy of ~50 us)
        key = (str(device), tuple(int(v) for v in sparse_tensor.spatial_shape))
        if key not in self._consts:
            shape = np.asarray(sparse_tensor.spatial_shape, dtype=np.float64)
            if self.voxel_extent is not None:
                unit = torch.tensor(self.voxel_extent / shape, dtype=torch.float32, device=device)
                extent = torch.tensor(self.voxel_extent, dtype=torch.float32, device=device)
            else:
                unit = torch.tensor(self.unit_voxel_extent, dtype=torch.float32, device=device)
                extent = torch.tensor(self.unit_voxel_extent * shape, dtype=torch.float32,
                                      device=device)
            self._consts[key] = (unit, extent)
        unit, extent = self._consts[key]
        centres = sparse_tensor.indices.float()
        centres[:, 1:] = centres[:, 1:] * unit - 0.5 * extent + 0.5 * unit
        return centres.contiguous().detach(), feat

    def _grid(self, sparse_tensor):
        """(unit, origin) of the voxel grid as float32 host arrays: the numbers the centres
        were computed from in _get_vertice_feats."""
        shape = np.asarray(sparse_tensor.spatial_shape, dtype=np.float64)
        if self.voxel_extent is not None:
            unit, extent = self.voxel_extent / shape, self.voxel_extent
        else:
            unit, extent = self.unit_voxel_extent, self.unit_voxel_extent * shape
        unit = unit.astype(np.float32)
        extent = np.asarray(extent, dtype=np.float64).astype(np.float32)
        return unit, np.float32(-0.5) * extent

    def _get_point_feats(self, target_points, query_points, query_feats, sparse_tensor=None):
        indices = None if sparse_tensor is None else sparse_tensor.indices
        if indices is not None and target_points.is_cuda and indices.dtype == torch.int32 \
                and target_points.dtype == torch.float32:
            # the known points are voxel centres: search around each point's own cell
            unit, origin = self._grid(sparse_tensor)
            dist2, idx = _ext.three_nn_grid(target_points, query_points, indices.contiguous(),
                                            sparse_tensor.batch_size,
                                            # (a point on the upper face of the grid has
                                            # voxel index == shape, voxelize.py:85-86)
                                            [int(v) + 1 for v in sparse_tensor.spatial_shape],
                                            origin, unit)
            dist = torch.sqrt(dist2)
        else:
            dist, idx = three_nn(target_points, query_points)
        dist_recip = 1.0 / (dist + 1e-8)
        norm = torch.sum(dist_recip, dim=1, keepdim=True)
        weight = dist_recip / norm
        return three_interpolate(query_feats.contiguous(), idx, weight.contiguous())
