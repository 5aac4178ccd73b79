"""Rasterize operator: the reference's Python surface over the gfx950 library.

Mirrors d3sim/algos/d3gs/render.py: the dataclasses (35-150), ``GaussianSplatOp``
with ``forward`` (169-1015), ``rasterize_forward_backward`` (1329-2316) and
``backward`` (2779-3374), the autograd glue (3376-3587) and the user entry point
``rasterize_gaussians`` (3783-3838).  Where the reference assembles CUDA source
text and JIT-compiles it, this module allocates with torch and calls the
ahead-of-time HIP library through ``_capi`` on torch's current stream.

Scope: single cameras and camera bundles (one pass over B x N render items), every
early filter (OBB_DFVT computed as the OBB tile set), RGB / RGBA / depth / custom
feature channels in NHWC or NCHW, instances, sparse mode, both backward algorithms.
``render_inv_depth`` keeps the reference's behaviour (1 / z is also what the lists are sorted by).
The few options outside that scope (``transmittance_is_double``, tile sizes other than
16 x 16, ``prep_user_inputs``) raise ``NotImplementedError``.
"""
from __future__ import annotations

import contextlib
import copy
import ctypes as C
import dataclasses
import math
import os
import time
import types
import warnings
import weakref

import numpy as np
import torch

from . import _capi
from .camera import BasicPinholeCamera
from .config_def import GaussianSplatConfig, RasterizeBackwardAlgo
from .model import GaussianModelOriginBase, GaussianModelOriginFused


def div_up(a: int, b: int) -> int:
    return (a + b - 1) // b


# Parity tests compare the sorted keys with the oracle's; they switch this on (through the environment, before the
# package is imported) so that an operator keeps the last view's sorted tile keys and indices alive.
KEEP_SORTED_KEYS = os.environ.get("D3GS_KEEP_SORTED_KEYS", "0") not in ("", "0")
# How long the host polls the pinned pair-count word before it falls back to synchronising the stream, and the
# largest view (in pairs the buffers are sized for) whose count is polled at all.
POLL_SECONDS = 0.02
POLL_MAX_PAIRS = 1 << 26


def poll_host_word(word, pending, seconds, synchronize, clock=time.perf_counter):
    """Waits until ``word[0]`` (a pinned host word a kernel stores into) no longer holds ``pending``.  Returns
    "polled" when the store showed up within ``seconds``; otherwise calls ``synchronize()`` (the stream has then run
    dry) and returns "synced" when the word has changed by then, "never" when it still holds ``pending``."""
    give_up = clock() + seconds
    while int(word[0]) == pending:
        if clock() > give_up:
            synchronize()
            return "never" if int(word[0]) == pending else "synced"
    return "polled"


@dataclasses.dataclass
class _StreamSlot:
    """What one forward pass at a time needs outside its own buffers, kept per (device, stream): the pinned host
    words the kernels report into (the pair count; the two sorts' status on the launch-by-launch path), the pair
    buffer size learnt from the stream's last view, and the side stream of the SH colours.  Two forwards of one
    operator on two streams use two slots; two host threads on ONE stream would still race."""
    count_host: torch.Tensor
    count_np: np.ndarray            # the same word, read without a tensor operation
    sort_status_host: torch.Tensor
    pair_capacity: int = 0
    poll_timeouts: int = 0          # consecutive views whose count did not arrive within the polling time
    side_stream: torch.cuda.Stream | None = None


@dataclasses.dataclass
class GaussianSplatOpContext:
    """render.py:57-72"""
    conic_opacity: torch.Tensor
    radii: torch.Tensor
    uvs: torch.Tensor
    rgb_gaussian: torch.Tensor | None
    gaussian_idx_sorted: torch.Tensor
    workload_ranges: torch.Tensor
    image_shape_wh: tuple[int, int]
    depths: torch.Tensor
    cov2d_vecs: torch.Tensor | None = None
    sh_to_rgb_ne_0: torch.Tensor | None = None
    # rasterize_backward_algo = PER_GAUSSIAN (render.py:44-55, 940-962): (bucket_offsets [tiles + 1] int32,
    # snapshots [buckets, 256, 4] float32), the running state of every pixel in front of each bucket of 64 list
    # entries, stored by the forward blend for the per-gaussian backward
    per_gaussian_snap: tuple | None = None
    # not in the reference: tile ids by descending list length, the blend kernels' launch order
    tile_order: torch.Tensor | None = None
    # not in the reference: the backward's [N, 16] gradient records, cleared by the forward blend kernel
    # (consumed by the first backward over this context)
    grad_records: torch.Tensor | None = None
    # float32 pool for the model gradients of this view, cleared with the records (see _grad_views)
    grad_pool: torch.Tensor | None = None
    # the allocation behind grad_records and grad_pool, until the forward blend has been asked to clear it
    grad_clear: torch.Tensor | None = None
    # one byte per gaussian, set by the blend backward where a record received anything (cleared with the records)
    grad_touched: torch.Tensor | None = None
    # custom feature channels of this view ([N, F]) kept for the backward pass
    custom_features: torch.Tensor | None = None
    # disable_builtin_rgb: the image in the kernels' own layout ([1, H, W, 3 or 4], colour channels zero); the
    # caller sees its alpha channel, or no channel at all, as out.color
    kernel_color: torch.Tensor | None = None
    # instance rendering: the view's camera in every instance frame ([I, 12] float32) and the int32 ids
    instance_cameras: torch.Tensor | None = None
    instance_ids: torch.Tensor | None = None
    # camera bundle rendered in one pass (render.py:314-326): B cameras, every per-gaussian array above has
    # B * N rows (item b * N + g), tile ids and ranges cover B * tiles; the [B, 16] camera table on the device
    batch_size: int = 1
    batch_cameras: torch.Tensor | None = None
    # sparse mode (render.py:234-238, 478-500): every per-gaussian array above has one row per ACCEPTED gaussian;
    # the gaussian of each row (int32 [V], ascending)
    sparse_gaussian_ids: torch.Tensor | None = None
    # ... and, for a bundle rendered in one pass, the camera of each row (int32 [V])
    sparse_batch_ids: torch.Tensor | None = None


@dataclasses.dataclass
class GaussianSplatOpBatchContext:
    """Context of a camera bundle with more than one camera: the cameras are rendered one after the
    other, each keeping its own single-camera context (None where nothing was rendered)."""
    per_camera: list
    cameras: list
    image_shape_wh: tuple[int, int]
    # sparse mode: rows of out.radii / out.sparse_gaussian_ids each camera contributed (also for a camera whose
    # accepted gaussians ended without a single pair, which has rows but no context)
    rows_per_camera: list | None = None


@dataclasses.dataclass
class GaussianSplatOutput:
    """render.py:74-100"""
    custom_features: torch.Tensor | None
    T: torch.Tensor
    color: torch.Tensor
    depth: torch.Tensor | None = None
    n_contrib: torch.Tensor | None = None
    radii: torch.Tensor | None = None
    sparse_gaussian_ids: torch.Tensor | None = None
    sparse_batch_ids: torch.Tensor | None = None

    @property
    def image_shape_wh(self) -> tuple[int, int]:
        return (self.T.shape[2], self.T.shape[1])

    def select_batch(self, batch_idx: int):
        s = slice(batch_idx, batch_idx + 1)
        return GaussianSplatOutput(
            custom_features=None if self.custom_features is None else self.custom_features[s],
            T=self.T[s], color=self.color[s], depth=None if self.depth is None else self.depth[s],
            n_contrib=None if self.n_contrib is None else self.n_contrib[s], radii=self.radii)


@dataclasses.dataclass
class RasterizeGradientOutput:
    """render.py:103-111"""
    duv: torch.Tensor
    dconic: torch.Tensor
    dopacity: torch.Tensor
    dcolor: torch.Tensor | None
    dcustom_features: torch.Tensor | None = None
    dz: torch.Tensor | None = None
    # not in the reference: the [N, 16] buffer the tensors above are strided views of
    records: torch.Tensor | None = None
    # not in the reference: one byte per gaussian, non-zero where the record received anything (or None)
    touched: torch.Tensor | None = None


@dataclasses.dataclass
class GaussianSplatGradients:
    """render.py:113-120"""
    drgb: torch.Tensor
    dT: torch.Tensor
    ddepth: torch.Tensor | None = None
    dcustom_features: torch.Tensor | None = None


@dataclasses.dataclass
class CameraParamBundle:
    focal_xy_ppoint: torch.Tensor
    image_shape_wh: tuple[int, int]
    frame_ids: torch.Tensor | None


@dataclasses.dataclass
class CameraBundle(CameraParamBundle):
    """render.py:129-150."""
    cam2world_T: torch.Tensor = None

    def __len__(self):
        return int(self.cam2world_T.shape[0])

    def select(self, b: int) -> "CameraBundle":
        return CameraBundle(self.focal_xy_ppoint[b:b + 1], self.image_shape_wh,
                            None if self.frame_ids is None else self.frame_ids[b:b + 1], self.cam2world_T[b:b + 1])

    @classmethod
    def from_pinhole_cams(cls, cams: list[BasicPinholeCamera], device="cuda"):
        c2w = np.stack([np.ascontiguousarray(c.pose.to_world[:3].T) for c in cams], 0).reshape(-1, 4, 3)
        fpp = np.stack([np.concatenate([c.focal_length, c.principal_point]) for c in cams], 0).reshape(-1, 4)
        return cls(torch.from_numpy(fpp.astype(np.float32)).to(device), cams[0].image_shape_wh, None,
                   torch.from_numpy(c2w.astype(np.float32)).to(device))


class GaussianSplatOp:
    """render.py:152-159: one op per config; the config is frozen at construction."""

    def __init__(self, cfg: GaussianSplatConfig) -> None:
        self._cfg = copy.deepcopy(cfg)
        self._lib = _capi.lib()  # fails loudly when the HIP library is not built
        self._check_supported()
        # optional per-stage timing: set to a dict to collect torch.cuda.Event pairs
        self.stage_events: dict[str, list] | None = None
        self.last_num_rendered = 0
        self.last_forward_fused = False
        self.rebin_count = 0        # views that outgrew the pair buffers sized from the previous view
        # The SH colours are only read by the blend, so they are computed on a second stream beside the
        # latency-bound sort stages.  Set to False for a single-stream forward (the fused preprocess).
        self.overlap_sh_colors = True
        # size the pair buffers from the previous view's count instead of waiting for this view's
        self.speculative_pair_buffers = True
        # the binning of such a view (depth order .. tile ranges) goes out as one library call
        self.fused_binning = True
        # training: the model-gradient arrays are allocated with the forward pass and cleared by its blend kernel
        self.clear_gradients_early = True
        # a CameraBundle of several cameras goes through the kernels in one pass (False: camera by camera)
        self.bundle_in_one_pass = True
        # ... and its preprocess backward in one launch (False: one launch per camera, each adding to the last)
        self.bundle_k9_in_one_launch = True
        # custom feature channels through the library's feature kernels (False: three at a time through the colour
        # kernels, one forward and one backward blend per triple)
        self.feature_kernels = True
        # the one-call binning carries the pairs' tile ids as 16-bit keys when the view has at most 2^16 tiles
        self.narrow_tile_keys = True
        # the one-call binning writes the pair count to its pinned host word with a store the host can see while
        # the stream runs on, and the host polls that word: an event recorded behind the binning would hold the
        # forward blend back by the few microseconds the stream takes to process the marker
        self.poll_pair_count = True
        self.recovered_views = 0    # views binned a second time because a look-back of the one-call binning gave up
        self._slots: dict[tuple[int, int], _StreamSlot] = {}
        self._last_sorted = None

    # ------------------------------------------------------------------ utils
    def _check_supported(self):
        c = self._cfg
        unsupported = {
            "tile_size != (16, 16)": tuple(c.tile_size) != (16, 16),
            "transmittance_is_double": c.transmittance_is_double,
            # sparse mode is built for the plain colour path (the reference itself excludes custom features there,
            # render.py:238)
            "sparse_mode with disable_builtin_rgb / PER_GAUSSIAN":
                c.sparse_mode and (c.disable_builtin_rgb
                                   or c.rasterize_backward_algo == RasterizeBackwardAlgo.PER_GAUSSIAN),
            # builtin colours off: the kernels blend zeros in their place (render.py:262, 662, 1898-1931)
            "disable_builtin_rgb with use_nchw": c.disable_builtin_rgb and c.use_nchw,
            # the per-gaussian backward (render.py:2319-2776) needs the model's own colours in the colour channels
            "rasterize_backward_algo = PER_GAUSSIAN with disable_builtin_rgb":
                c.rasterize_backward_algo == RasterizeBackwardAlgo.PER_GAUSSIAN and c.disable_builtin_rgb,
            # Accepted without a code path of their own, because they change how the reference computes and not
            # what: move_opacity_in_grad_to_prep (render.py:1973-1990, 2995-3003) takes the factors opacity, -1/2
            # and -1 out of the per-pixel gradient terms and applies them once per gaussian -- the same gradient up
            # to rounding; the blend backward here applies the conic factors once per tile and gaussian in any
            # case, and taking the opacity out as well measured no gain; use_int64_tile_touched (render.py:657-660)
            # widens the tile counters, while the reference's sort takes an int count all the same; this build
            # keeps 31-bit list positions and raises beyond 2^31 - 1024 pairs per call
        }
        bad = [k for k, v in unsupported.items() if v]
        if bad:
            raise NotImplementedError("GaussianSplatOp (gfx950 build): unsupported config options: " + ", ".join(bad))

    @property
    def _last_keys_sorted(self) -> torch.Tensor:
        """The reference's sorted 64-bit keys, (tile << 32) | depth bits, rebuilt from the last forward's
        sorted tile keys and gaussian indices (parity tests compare them with the oracle's)."""
        assert self._last_sorted is not None, "set D3GS_KEEP_SORTED_KEYS=1 before importing the package"
        tile_keys, idx, depths = self._last_sorted
        if tile_keys.dtype == torch.int16:      # the one-call binning's 16-bit tile ids
            tile_keys = tile_keys.long() & 0xFFFF
        if self._cfg.enable_32bit_sort:     # render.py:767-770, 820: (tile << 18) | depth steps
            steps = (depths / torch.tensor(self._cfg.depth_32bit_prec, dtype=torch.float32, device=depths.device))
            return (tile_keys.long() << 18) | (steps.long()[idx.long()] & 0x3FFFF)
        bits = depths.view(torch.int32)[idx.long()].long() & 0xFFFFFFFF
        return (tile_keys.long() << 32) | bits

    @property
    def is_nchw(self):
        return self._cfg.use_nchw

    @property
    def is_rgba(self):
        return self._cfg.render_rgba

    @contextlib.contextmanager
    def _stage(self, name: str):
        if self.stage_events is None:
            yield
            return
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        yield
        b.record()
        self.stage_events.setdefault(name, []).append((a, b))

    @staticmethod
    def _stream():
        """The current stream's handle.  (torch.cuda.current_stream() builds a Stream object, some 10 us of host
        time a call, which a view of a small scene notices: its host code is what bounds it.)"""
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:
            return C.c_void_p(raw(torch.cuda.current_device()))
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def _camera_arrays(self, cameras):
        if isinstance(cameras, BasicPinholeCamera):
            intrinsic = cameras.intrinsic
            focal = np.array([intrinsic[0, 0], intrinsic[1, 1]], np.float32)
            pp = np.array([intrinsic[0, 2], intrinsic[1, 2]], np.float32)
            c2w_T = np.ascontiguousarray(np.asarray(cameras.pose.to_world)[:3].T).astype(np.float32)
        elif isinstance(cameras, CameraBundle):
            if cameras.cam2world_T.shape[0] != 1:
                # several cameras: the kernels read them from the device table (see batch_table); nothing is
                # brought to the host
                return None, None, None, cameras.image_shape_wh
            fpp = cameras.focal_xy_ppoint[0].detach().cpu().numpy().astype(np.float32)
            focal, pp = fpp[:2], fpp[2:]
            c2w_T = cameras.cam2world_T[0].detach().cpu().numpy().astype(np.float32).reshape(4, 3)
        else:
            raise TypeError(f"unsupported camera type {type(cameras)}")
        return focal, pp, c2w_T, cameras.image_shape_wh

    def instance_table(self, model, cameras, instance2world_T):
        """Instance rendering (render.py:207-220, 346-356): gaussians with ``model.instance_id[i] = k >= 0`` live
        in the frame of object instance k, whose pose this frame is ``instance2world_T[frame][k]`` ([4, 3]: three
        rows holding the columns of the rotation, then the translation; rigid).  The reference composes
        cam2instance = world2instance o cam2world per gaussian inside its kernels; here it is done once per
        instance, in float64 on the device, and the kernels read a [I, 12] float32 table: the world-to-camera
        rotation in the instance frame (row major) and the camera centre in the instance frame.
        Returns ``(instance_ids int32 [N], instance_cameras float32 [I, 12])``; for a bundle of B > 1 cameras
        the table has B * I rows, the I rows of camera 0 first (each camera with the poses of its own frame)."""
        assert model.instance_id is not None, "instance_id must be provided in model when render with instance"
        T = instance2world_T
        if T.ndim == 4:      # [num_frame, num_instance, 4, 3]
            if isinstance(cameras, BasicPinholeCamera):
                assert cameras.frame_local_id is not None, "frame_local_id must be set when render with instance"
                T = T[int(cameras.frame_local_id)]
            else:
                assert cameras.frame_ids is not None, "frame_ids must be provided when render with instance"
                T = T[cameras.frame_ids[0].to(device=T.device, dtype=torch.long)]
        assert T.ndim == 3 and tuple(T.shape[1:]) == (4, 3), \
            "instance2world_T must be [num_frame, num_instance, 4, 3] (or [num_instance, 4, 3] for one frame)"
        dev = model.xyz.device
        ids = model.instance_id.detach().to(device=dev, dtype=torch.int32).contiguous()
        assert ids.numel() == len(model), "instance_id must hold one id per gaussian"
        if isinstance(cameras, CameraBundle) and len(cameras) > 1:
            Tall = instance2world_T
            if Tall.ndim == 4:
                assert cameras.frame_ids is not None, "frame_ids must be provided when render with instance"
                Tall = Tall[cameras.frame_ids.to(device=Tall.device, dtype=torch.long)]      # [B, I, 4, 3]
            else:
                Tall = Tall.unsqueeze(0).expand(len(cameras), -1, -1, -1)
            assert Tall.ndim == 4 and tuple(Tall.shape[2:]) == (4, 3), "instance2world_T must be [num_frame, num_instance, 4, 3]"
            Tall = Tall.detach().to(device=dev, dtype=torch.float64)
            cw = cameras.cam2world_T.detach().to(device=dev, dtype=torch.float32).reshape(-1, 4, 3).to(torch.float64)
            rot_T = Tall[:, :, :3, :]                                              # [B, I, 3, 3]
            w2c = cw[:, None, :3, :] @ rot_T.transpose(2, 3)
            centre = rot_T @ (cw[:, None, 3, :] - Tall[:, :, 3, :]).unsqueeze(-1)
            table = torch.cat([w2c.reshape(-1, 9), centre.reshape(-1, 3)], 1).to(torch.float32).contiguous()
            return ids, table
        T = T.detach().to(device=dev, dtype=torch.float64)
        cw = torch.from_numpy(self._camera_arrays(cameras)[2].astype(np.float64)).to(dev)
        rot_T = T[:, :3, :]                                   # R_i^T: world -> instance
        w2c = cw[:3] @ rot_T.transpose(1, 2)                  # R_c^T R_i
        centre = rot_T @ (cw[3] - T[:, 3, :]).unsqueeze(-1)   # R_i^T (c - t_i)
        table = torch.cat([w2c.reshape(-1, 9), centre.reshape(-1, 3)], 1).to(torch.float32).contiguous()
        return ids, table

    @staticmethod
    def _instances_arg(ids, table, batch=1, camera=None):
        """The kernels' instance argument; `table` holds `batch` tables one after the other, of which `camera`
        selects one (the preprocess backward runs camera by camera)."""
        if table is None:
            return None
        count = int(table.shape[0]) // batch
        first = 0 if camera is None else camera * count
        return C.byref(_capi.Instances(ids.data_ptr(), table.data_ptr() + 48 * first, count))

    @staticmethod
    def batch_table(cameras: "CameraBundle", device) -> torch.Tensor:
        """The cameras of a bundle as the [B, 16] float32 device table the kernels read (render.py:316-323 loads
        the same values from cam2world_T [B, 4, 3] and focal_xy_ppoint [B, 4]): rows 0-2 of cam2world_T, its row 3
        (the centre), focal x, y, principal point x, y.  Built on the device; nothing is read back."""
        c2w = cameras.cam2world_T.detach().to(device=device, dtype=torch.float32).reshape(-1, 4, 3)
        fpp = cameras.focal_xy_ppoint.detach().to(device=device, dtype=torch.float32).reshape(-1, 4)
        assert c2w.shape[0] == fpp.shape[0], "cam2world_T and focal_xy_ppoint must hold one row per camera"
        return torch.cat([c2w[:, :3, :].reshape(-1, 9), c2w[:, 3, :], fpp], dim=1).contiguous()

    def make_params(self, model: GaussianModelOriginBase, cameras, training: bool, batch_cameras=None) -> _capi.Params:
        """Scalars the reference bakes into kernel source (render.py:198-230, 333-358).  With ``batch_cameras``
        (the [B, 16] device table of a bundle of B > 1 cameras) the per-camera fields stay zero: the kernels take
        them from the table."""
        c = self._cfg
        focal, pp, c2w_T, (width, height) = self._camera_arrays(cameras)
        P = _capi.Params()
        P.n = len(model)
        P.width, P.height = int(width), int(height)
        P.tiles_x, P.tiles_y = div_up(width, 16), div_up(height, 16)
        P.sh_degree = int(model.cur_sh_degree)
        P.sh_stride = int(model.color_sh.shape[1])
        P.has_sh_base = int(model.color_sh_base is not None)
        P.filter_algo = int(c.early_filter_algo)
        P.training = int(bool(training))
        if batch_cameras is not None:
            assert focal is None and batch_cameras.dtype == torch.float32 and batch_cameras.is_contiguous() \
                and batch_cameras.shape[1] == _capi.BATCH_CAMERA_FLOATS
            P.batch_size = int(batch_cameras.shape[0])
            P.batch_cameras = batch_cameras.data_ptr()
        else:
            assert focal is not None, "a bundle of several cameras needs its device table (batch_table)"
            P.fx, P.fy, P.cx, P.cy = float(focal[0]), float(focal[1]), float(pp[0]), float(pp[1])
            tan_fov = np.float32(0.5) * np.array([width, height], np.float32) / focal
            P.tan_fovx, P.tan_fovy = float(tan_fov[0]), float(tan_fov[1])
            P.w2c[:] = [float(v) for v in c2w_T[:3].reshape(-1)]
            P.cam_center[:] = [float(v) for v in c2w_T[3]]
        P.z_near, P.z_far, P.eps = float(c.near), float(c.far), float(c.eps)
        P.radii_eigen_eps = float(c.cov2d_radii_eigen_eps)
        P.clamp_factor = float(c.projected_clamp_factor)
        P.std_sigma = float(c.gaussian_std_sigma)
        P.lowpass = float(c.gaussian_lowpass_filter)
        P.alpha_eps = float(c.alpha_eps)
        P.transmittance_eps = float(c.transmittance_eps)
        P.scale_global = float(c.scale_global)
        P.bg[:] = [float(v) for v in np.asarray(c.bg_color, np.float32).reshape(3)]
        # a fused model hands over raw tensors; any other family has applied its activations in torch
        P.fused_activation = int(isinstance(model, GaussianModelOriginFused))
        P.render_depth, P.render_rgba = int(c.render_depth), int(c.render_rgba)
        P.use_nchw, P.enable_anti_aliasing = int(c.use_nchw), int(c.enable_anti_aliasing)
        P.enable_32bit_sort, P.depth_32bit_prec = int(c.enable_32bit_sort), float(c.depth_32bit_prec)
        # 1 / z in the depth buffer (render.py:582); as in the reference that buffer also gives the sort key its depth
        # part (render.py:773), so the lists then run from the far end to the near one
        P.render_inv_depth = int(c.render_inv_depth)
        if c.enable_32bit_sort:
            assert P.tiles_x * P.tiles_y * max(P.batch_size, 1) < 2 ** 14, "32bit sort only support 14 bits tile idx"   # render.py:227-228
        return P

    @staticmethod
    def _check_model(model: GaussianModelOriginBase):
        n = len(model)
        exp = {"xyz": (n, 3), "quaternion_xyzw": (n, 4), "scale": (n, 3), "opacity": (n,)}
        for name, shape in exp.items():
            t = getattr(model, name)
            assert t.is_cuda and t.dtype == torch.float32 and tuple(t.shape) == shape and t.is_contiguous(), \
                f"model.{name} must be a contiguous float32 cuda tensor of shape {shape}"
        sh = model.color_sh
        assert sh.is_cuda and sh.dtype == torch.float32 and sh.ndim == 3 and sh.shape[0] == n and sh.shape[2] == 3 \
            and sh.is_contiguous(), "model.color_sh must be a contiguous float32 cuda tensor [N, K, 3]"
        if model.color_sh_base is not None:
            b = model.color_sh_base
            assert b.is_cuda and b.dtype == torch.float32 and tuple(b.shape) == (n, 3) and b.is_contiguous()
        assert 0 <= model.cur_sh_degree <= min(3, model.color_sh_degree), "cur_sh_degree out of range"

    @staticmethod
    def _params_signature(model, cameras):
        """What the kernel parameters of a view depend on, cheap to form: backward() reuses the forward's parameters
        only while this has not changed (a pose updated in place, a model grown or pruned, a raised SH degree)."""
        if isinstance(cameras, BasicPinholeCamera):
            cam = (np.asarray(cameras.intrinsic).tobytes(), np.asarray(cameras.pose.to_world).tobytes(),
                   tuple(cameras.image_shape_wh))
        else:
            cam = tuple((t.data_ptr(), t._version, tuple(t.shape)) for t in (cameras.cam2world_T, cameras.focal_xy_ppoint)) \
                + (tuple(cameras.image_shape_wh),)
        return (len(model), int(model.cur_sh_degree), int(model.color_sh.shape[1]), model.color_sh_base is not None,
                type(model).__name__, cam)

    def _snapshot_floats(self) -> int:
        """Floats per pixel and bucket of the per-gaussian backward's snapshots: T and the colour accumulated so far,
        and with a depth or an alpha channel a second quad with their sums (render.py:1744-1759, 2412-2415)."""
        return 8 if (self._cfg.render_depth or self._cfg.render_rgba) else 4

    # ---------------------------------------------------------------- forward
    def forward(self, model: GaussianModelOriginBase, cameras, training: bool = False, instance2world_T=None,
                custom_features=None, mask=None, prep_user_inputs=None):
        """render.py:169-1015.  Returns ``(GaussianSplatOutput, GaussianSplatOpContext | None)``.

        The pass runs in four steps, each a method of its own: ``_start_view`` (arguments, kernel parameters, sparse
        mode's first pass), ``_preprocess`` (K1 and the colours), ``_order_and_count`` (depth order and pair count, or
        the whole binning as one library call) and ``_bin_and_blend`` (key expansion .. forward blend); ``forward``
        strings them together and decides, once the pair count has reached the host, whether the view has to be
        binned again (buffers outgrown, or a look-back that gave up)."""
        assert model.act_applied, "model must be activated before render"
        batch = len(cameras) if isinstance(cameras, CameraBundle) else 1
        if batch != 1 and not self._bundle_in_one_pass(batch, cameras):
            return self._forward_bundle(model, cameras, training, instance2world_T, custom_features, mask,
                                        prep_user_inputs)
        if prep_user_inputs:
            raise NotImplementedError("prep_user_inputs is not supported")
        v = self._start_view(model, cameras, training, instance2world_T, custom_features, mask, batch)
        if v.sparse and v.n == 0:      # nothing accepted: the empty render, without touching zero-row buffers
            self.last_num_rendered = 0
            self._alloc_outputs(v)
            return self._empty_result(v)
        self._alloc_zero_workspaces(v, v.slot.pair_capacity if self.speculative_pair_buffers else 0)
        self._preprocess(v)
        self._order_and_count(v)
        self._alloc_outputs(v)

        # The reference reads the pair count back before it can size the key buffers (render.py:695),
        # which idles the GPU for a host round trip.  From the second view on the buffers are sized from
        # the previous count with head room, everything is enqueued at once and the count is read
        # afterwards; a view that outgrows its buffers is binned again with exact sizes.
        capacity = v.spec_capacity
        ctx = None
        if capacity > 0:
            ctx, tile_keys_sorted = self._bin_and_blend(v, capacity, True)
        num_rendered = self._wait_pair_count(v)
        if num_rendered in (_capi.COUNT_SORT_GAVE_UP, _capi.COUNT_SCAN_GAVE_UP) and v.fused:
            # A look-back of the one-call binning ran out of its bounded wait (its workgroups rely on being
            # dispatched in id order): nothing of this binning is used; the view is binned once more, launch by
            # launch into exactly sized buffers, before anything is raised.
            self.recovered_views += 1
            ctx = None
            self._alloc_zero_workspaces(v, 0)
            self._preprocess(v)       # (its depth keys were sorted in place by the binning that failed)
            self._order_and_count(v, stepwise=True)
            num_rendered = self._wait_pair_count(v)
        if num_rendered == _capi.COUNT_SORT_GAVE_UP:
            raise RuntimeError("d3gs_bin_pairs: a sort workgroup's bounded wait on an earlier tile ran out; "
                               "the tile lists are not sorted")
        if num_rendered < 0:
            raise RuntimeError("d3gs_scan_gathered: a workgroup's bounded wait on an earlier chunk ran out")
        if not v.fused:
            self._check_sort_status(v, 0, "depth order")
        if num_rendered > _capi.MAX_PAIRS:
            raise RuntimeError(f"GaussianSplatOp: {num_rendered} (tile, gaussian) pairs in one call; list positions are "
                               f"31-bit, at most {_capi.MAX_PAIRS} pairs (render fewer cameras per bundle, or use a "
                               "tighter early_filter_algo)")
        self.last_num_rendered = num_rendered
        v.slot.pair_capacity = min(num_rendered + num_rendered // 4 + 4096, _capi.MAX_PAIRS)
        if num_rendered == 0:
            return self._empty_result(v)
        if ctx is None or num_rendered > capacity:
            self.rebin_count += int(ctx is not None)
            ctx, tile_keys_sorted = self._bin_and_blend(v, num_rendered, False)
        if v.pair_sort_done is not None:
            # everything is enqueued; the host only waits for the pair sort's status word, the blend runs on
            v.pair_sort_done.synchronize()
            self._check_sort_status(v, 1, "tile lists")
        ctx.gaussian_idx_sorted = ctx.gaussian_idx_sorted[:num_rendered]
        out = v.out
        if custom_features is not None:
            out.custom_features = self._blend_custom_features(v.P, ctx, out, custom_features)
            ctx.custom_features = custom_features
        if KEEP_SORTED_KEYS:        # parity tests rebuild the reference's 64-bit keys from these
            self._last_sorted = (tile_keys_sorted[:num_rendered], ctx.gaussian_idx_sorted, v.depths)
        if not training:
            ctx = None
        return out, ctx

    # -- step 1: arguments, parameters, per-stream state, sparse mode's first pass
    def _slot(self, dev) -> _StreamSlot:
        """The host words and hints of the stream this call runs on (one set per device and stream: two forwards of
        one operator on two streams do not share a word)."""
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        handle = raw(torch.cuda.current_device()) if raw is not None else torch.cuda.current_stream().cuda_stream
        key = (dev.index if dev.index is not None else torch.cuda.current_device(), int(handle))
        slot = self._slots.get(key)
        if slot is None:
            count_host = torch.empty(1, dtype=torch.int64, pin_memory=True)
            slot = _StreamSlot(count_host=count_host, count_np=count_host.numpy(),
                               sort_status_host=torch.zeros(2, dtype=torch.int32, pin_memory=True))
            self._slots[key] = slot
        return slot

    def _start_view(self, model, cameras, training, instance2world_T, custom_features, mask, batch):
        self._check_model(model)
        if custom_features is not None:
            assert not self.is_nchw, "custom feat don't support nchw, set use_nchw=False in config."   # render.py:246
            # one row per (camera, gaussian), camera by camera (render.py:245)
            assert custom_features.is_cuda and custom_features.dtype == torch.float32 and custom_features.ndim == 2 \
                and custom_features.shape[0] == batch * len(model) and custom_features.is_contiguous(), \
                "custom_features must be a contiguous float32 cuda tensor [B * N, F]"
        if mask is not None:
            # True rejects the gaussian (render.py:306-308); one entry per (camera, gaussian)
            assert mask.is_cuda and mask.dtype in (torch.bool, torch.uint8) and mask.numel() == batch * len(model) \
                and mask.is_contiguous(), "mask must be a contiguous bool/uint8 cuda tensor with one entry per gaussian"
            if mask.dtype == torch.bool:
                mask = mask.view(torch.uint8)
        L = self._lib
        v = types.SimpleNamespace()
        v.model, v.cameras, v.training, v.batch, v.mask, v.custom_features = model, cameras, bool(training), batch, mask, custom_features
        v.dev = dev = model.xyz.device
        v.batch_cams = self.batch_table(cameras, dev) if batch > 1 else None
        v.P = P = self.make_params(model, cameras, training, v.batch_cams)
        v.inst_ids = v.inst_cams = None
        if instance2world_T is not None:
            v.inst_ids, v.inst_cams = self.instance_table(model, cameras, instance2world_T)
        v.inst = self._instances_arg(v.inst_ids, v.inst_cams, batch)
        # n: render items = gaussians x cameras (item b * N + g is gaussian g seen by camera b); everything the
        # preprocess writes has one row per item, the tile ids carry the camera
        v.n = P.n * batch
        v.width, v.height = P.width, P.height
        v.num_tiles = P.tiles_x * P.tiles_y * batch
        v.s = self._stream()
        v.slot = self._slot(dev)
        v.tile_bits = L.d3gs_higher_msb(v.num_tiles)
        v.depth_bits = L.d3gs_depth_key_bits(C.byref(P))      # the depth sort's key width: 27 bits for the default planes
        v.status_pending, v.pair_sort_done, v.pooled_ranges_used = [], None, False
        # Sparse mode (render.py:234-238, 478-500, 622-640): a first pass of the preprocess flags the accepted
        # gaussians, a scan gives each its row, and from here on n is their number V: every buffer below has V rows
        # and the kernels after the preprocess see a scene of V gaussians.  The count has to reach the host before
        # anything can be sized (the reference reads it back the same way, render.py:636).
        v.sparse = bool(self._cfg.sparse_mode)
        v.Pd = P            # what the kernels behind the preprocess are given
        v.sparse_scan = v.sparse_gaussian_ids = v.sparse_batch_ids = None
        if v.sparse:
            assert custom_features is None, "custom_features must not be provided in sparse mode"    # render.py:238
            n, i32 = v.n, torch.int32
            flags = torch.empty(n, dtype=i32, device=dev)
            _capi.check(L.d3gs_preprocess_fwd_sparse(
                C.byref(P), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw), _capi.ptr(model.scale),
                _capi.ptr(model.opacity), _capi.ptr(mask), _capi.ptr(flags), *([None] * 11), v.inst, v.s),
                "d3gs_preprocess_fwd_sparse (flags)")
            v.sparse_scan = torch.empty(n, dtype=i32, device=dev)
            ws_bytes = C.c_size_t(0)
            _capi.check(L.d3gs_scan_gathered_workspace_bytes(n, C.byref(ws_bytes)), "d3gs_scan_gathered_workspace_bytes")
            ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=dev)
            total_valid = torch.empty(1, dtype=torch.int64, device=dev)
            _capi.check(L.d3gs_scan_gathered(_capi.ptr(flags), n, None, n, _capi.ptr(v.sparse_scan), _capi.ptr(ws),
                                             ws.numel(), 0, _capi.ptr(total_valid),
                                             C.c_void_p(v.slot.count_host.data_ptr()), v.s), "d3gs_scan_gathered (flags)")
            torch.cuda.current_stream().synchronize()
            num_valid = int(v.slot.count_host[0])
            if num_valid < 0:
                raise RuntimeError("d3gs_scan_gathered: a workgroup's bounded wait on an earlier chunk ran out")
            v.n = num_valid
            # what the kernels behind the preprocess see: V compact rows; a bundle keeps its camera count (tile ids
            # and images carry the camera) and says that its rows are compact
            v.Pd = _capi.Params.from_buffer_copy(P)
            v.Pd.n = num_valid
            if batch > 1:
                v.Pd.compact_items = num_valid
            else:
                v.Pd.batch_size, v.Pd.batch_cameras = 0, None
            v.sparse_gaussian_ids = torch.empty(num_valid, dtype=i32, device=dev)
            v.sparse_batch_ids = torch.empty(num_valid, dtype=i32, device=dev)
        return v

    def _sort_ws_bytes(self, count, begin_bit, end_bit):
        nbytes = C.c_size_t(0)
        _capi.check(self._lib.d3gs_sort_workspace_bytes(count, begin_bit, end_bit, C.byref(nbytes)),
                    "d3gs_sort_workspace_bytes")
        return nbytes.value

    def _alloc_zero_workspaces(self, v, spec_capacity):
        """Every zero-initialised work buffer of the forward pass comes out of one fill (the two sorts' and the
        scan's workspaces, the tile ranges), issued ahead of the preprocess so that nothing waits for it later."""
        v.spec_capacity = spec_capacity
        align = lambda x: (x + 255) // 256 * 256
        scan_ws_bytes = C.c_size_t(0)
        _capi.check(self._lib.d3gs_scan_gathered_workspace_bytes(v.n, C.byref(scan_ws_bytes)),
                    "d3gs_scan_gathered_workspace_bytes")
        sizes = [align(self._sort_ws_bytes(v.n, 0, v.depth_bits)),
                 align(self._sort_ws_bytes(spec_capacity, 0, v.tile_bits)) if spec_capacity else 0,
                 align(v.num_tiles * 8), align(scan_ws_bytes.value)]
        zero_pool = torch.zeros(sum(sizes), dtype=torch.uint8, device=v.dev)
        v.zero_scan_ws = zero_pool[sum(sizes[:3]):]
        v.zero_ws_n = zero_pool[:sizes[0]]
        v.zero_ws_m = zero_pool[sizes[0]:sizes[0] + sizes[1]] if spec_capacity else None
        v.zero_ranges = zero_pool[sizes[0] + sizes[1]:sizes[0] + sizes[1] + v.num_tiles * 8].view(torch.int32).view(v.num_tiles, 2)
        v.pooled_ranges_used = False

    # -- step 2: K1 and the colours
    def _preprocess(self, v):
        L, P, model, dev, n, s = self._lib, v.P, v.model, v.dev, v.n, v.s
        f32, i32 = torch.float32, torch.int32
        training, sparse, mask = v.training, v.sparse, v.mask
        with self._stage("preprocess"):
            v.depths = depths = torch.empty(n, dtype=f32, device=dev)
            v.radii = radii = torch.empty(n, dtype=i32, device=dev)
            v.uvs = uvs = torch.empty((n, 2), dtype=f32, device=dev)
            v.conic_opacity = conic_opacity = torch.empty((n, 4), dtype=f32, device=dev)
            v.tiles_touched = tiles_touched = torch.empty(n, dtype=i32, device=dev)
            v.rgb_gaussian = rgb_gaussian = torch.empty((n, 3), dtype=f32, device=dev)
            v.cov2d_vecs = cov2d_vecs = torch.empty((n, 3), dtype=f32, device=dev) if training else None
            v.ne0 = ne0 = torch.empty(n, dtype=torch.uint8, device=dev) if training else None
            # kept-tile record per gaussian: key expansion reads it instead of repeating the tile tests
            v.tile_masks = tile_masks = torch.empty((n, 2), dtype=torch.int64, device=dev)
            v.depth_keys = depth_keys = torch.empty(n, dtype=i32, device=dev)      # float bits of the depths: the depth sort's keys
            # The backward's accumulators (one record per gaussian) and, with clear_gradients_early, the model
            # gradient arrays: one allocation that the forward blend kernel clears while it runs (it leaves the
            # memory pipes idle).  Most gaussians of a view end with an all-zero gradient (culled, or never reached
            # before their pixels saturated), which the preprocess backward then need not write.
            v.grad_records = v.grad_pool = v.grad_clear = v.grad_touched = None
            if training:
                rec_floats = n * _capi.GRAD_RECORD_FLOATS
                pool_floats = self._grad_pool_floats(model) if self.clear_gradients_early else 0
                mark_floats = (n + 15) // 16 * 4          # n bytes, in whole 16-byte units
                if sparse:      # sparse gradients: one row per accepted gaussian (render.py:2918)
                    pool_floats = self._grad_pool_floats(model, n) if self.clear_gradients_early else 0
                v.grad_clear = torch.empty(rec_floats + pool_floats + mark_floats, dtype=f32, device=dev)
                # (bundle: one record per render item, one set of model gradient arrays)
                v.grad_records = v.grad_clear[:rec_floats].view(n, _capi.GRAD_RECORD_FLOATS)
                v.grad_pool = v.grad_clear[rec_floats:rec_floats + pool_floats] if pool_floats else None
                v.grad_touched = v.grad_clear[rec_floats + pool_floats:].view(torch.uint8)[:n]
            overlap = bool(self.overlap_sh_colors)
            v.no_rgb = no_rgb = bool(self._cfg.disable_builtin_rgb)
            if no_rgb:      # no SH evaluation: zero colours, nothing clamped
                rgb_gaussian.zero_()
                if ne0 is not None:
                    ne0.zero_()
            if sparse:       # second pass: the accepted gaussians' outputs, row by row in ascending order
                overlap = True      # (the colours always come from their own kernel here)
                _capi.check(L.d3gs_preprocess_fwd_sparse(
                    C.byref(P), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw), _capi.ptr(model.scale),
                    _capi.ptr(model.opacity), _capi.ptr(mask), None, _capi.ptr(v.sparse_scan),
                    _capi.ptr(v.sparse_gaussian_ids), _capi.ptr(v.sparse_batch_ids), _capi.ptr(depths), _capi.ptr(radii),
                    _capi.ptr(uvs), _capi.ptr(conic_opacity), _capi.ptr(tiles_touched), _capi.ptr(cov2d_vecs),
                    _capi.ptr(tile_masks), _capi.ptr(depth_keys), v.inst, s), "d3gs_preprocess_fwd_sparse")
            else:
                _capi.check(L.d3gs_preprocess_fwd(
                    C.byref(P), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw), _capi.ptr(model.scale),
                    _capi.ptr(model.opacity), _capi.ptr(model.color_sh), _capi.ptr(model.color_sh_base),
                    _capi.ptr(mask), _capi.ptr(depths), _capi.ptr(radii), _capi.ptr(uvs), _capi.ptr(conic_opacity),
                    _capi.ptr(tiles_touched), None if (overlap or no_rgb) else _capi.ptr(rgb_gaussian), _capi.ptr(cov2d_vecs),
                    None if (overlap or no_rgb) else _capi.ptr(ne0), _capi.ptr(tile_masks), _capi.ptr(depth_keys), v.inst, s),
                    "d3gs_preprocess_fwd")
        # The SH colours are only read by the blend: they run on a second (default-priority) stream beside the
        # latency-bound binning stages and are joined in front of the forward blend.
        v.sh_done = None
        if overlap:
            slot = v.slot
            if slot.side_stream is None or slot.side_stream.device != dev:
                slot.side_stream = torch.cuda.Stream(device=dev)   # default priority
            v.main_stream = main = torch.cuda.current_stream()
            side = slot.side_stream
            side.wait_stream(main)          # radii (and the buffers' allocation) are ready
            ta = torch.cuda.Event(enable_timing=True) if (self.stage_events is not None and not no_rgb) else None
            if ta is not None:
                ta.record(side)
            if sparse:
                _capi.check(L.d3gs_sh_colors_sparse(
                    C.byref(P), _capi.ptr(v.sparse_gaussian_ids), _capi.ptr(v.sparse_batch_ids), n, _capi.ptr(model.xyz),
                    _capi.ptr(model.color_sh), _capi.ptr(model.color_sh_base), _capi.ptr(radii), _capi.ptr(rgb_gaussian),
                    _capi.ptr(ne0), v.inst, C.c_void_p(side.cuda_stream)), "d3gs_sh_colors_sparse")
            elif not no_rgb:
                _capi.check(L.d3gs_sh_colors(
                    C.byref(P), _capi.ptr(model.xyz), _capi.ptr(model.color_sh), _capi.ptr(model.color_sh_base),
                    _capi.ptr(radii), _capi.ptr(rgb_gaussian), _capi.ptr(ne0), v.inst, C.c_void_p(side.cuda_stream)),
                    "d3gs_sh_colors")
            tb = torch.cuda.Event(enable_timing=True) if ta is not None else None
            if tb is not None:
                tb.record(side)
                self.stage_events.setdefault("sh_colors", []).append((ta, tb))
            v.sh_done = torch.cuda.Event()
            v.sh_done.record(side)

    # -- the radix sort of the launch-by-launch path and its status words
    def _sort(self, v, keys_a, vals_a, count, begin_bit, end_bit, count_dev=None, values_are_indices=False, zero_ws=None,
              status_slot=None):
        L, s = self._lib, v.s
        keys_b, vals_b = torch.empty_like(keys_a), torch.empty_like(vals_a)
        nbytes = self._sort_ws_bytes(count, begin_bit, end_bit)
        ws = zero_ws if zero_ws is not None else torch.empty(nbytes, dtype=torch.uint8, device=v.dev)
        assert ws.numel() >= nbytes
        in_b = C.c_int(0)
        if status_slot is not None:
            v.slot.sort_status_host[status_slot] = 0
        if keys_a.dtype == torch.int64:
            rc = L.d3gs_sort_pairs(_capi.ptr(keys_a), _capi.ptr(keys_b), _capi.ptr(vals_a), _capi.ptr(vals_b),
                                   _capi.ptr(ws), nbytes, count, begin_bit, end_bit, C.byref(in_b), s)
        else:
            rc = L.d3gs_sort_pairs_u32(_capi.ptr(keys_a), _capi.ptr(keys_b), _capi.ptr(vals_a), _capi.ptr(vals_b),
                                       _capi.ptr(ws), nbytes, count, count_dev, int(values_are_indices),
                                       int(zero_ws is not None), begin_bit, end_bit, C.byref(in_b), s)
        _capi.check(rc, "d3gs_sort_pairs")
        if status_slot is not None and count > 0 and end_bit > begin_bit:
            v.status_pending.append((ws, nbytes, count, begin_bit, end_bit, status_slot))
        return (keys_b, vals_b) if in_b.value else (keys_a, vals_a)

    def _report_sort_status(self, v):
        """The error word of every sort issued since the last call (a look-back that gave up) goes to its
        pinned host word, by a one-thread kernel behind the sort (outside the stage timers)."""
        while v.status_pending:
            ws, nbytes, count, begin_bit, end_bit, slot = v.status_pending.pop()
            _capi.check(self._lib.d3gs_sort_status(_capi.ptr(ws), nbytes, count, begin_bit, end_bit, None,
                                                   C.c_void_p(v.slot.sort_status_host.data_ptr() + 4 * slot), v.s),
                        "d3gs_sort_status")

    @staticmethod
    def _check_sort_status(v, slot, what):
        if int(v.slot.sort_status_host[slot]) != 0:
            raise RuntimeError(f"d3gs_sort_pairs_u32 ({what}): a workgroup's bounded wait on an earlier tile ran "
                               "out; the list is not sorted")

    # -- step 3: depth order and pair count (or the whole binning as one call)
    def _order_and_count(self, v, stepwise=False):
        """With buffers sized from the previous view and no stage timers, the whole binning is one call into the
        library (d3gs_bin_pairs): the launches of this phase are short, and issuing them one by one from Python
        leaves the GPU idle between them.  Otherwise (first view of a stream, stage timers, `stepwise`) the depth
        sort and the scan are issued here and the rest follows once the pair count is known."""
        L, dev, n, s = self._lib, v.dev, v.n, v.s
        i32 = torch.int32
        v.fused = bool(self.fused_binning and v.spec_capacity > 0 and self.stage_events is None and not stepwise)
        self.last_forward_fused = v.fused      # which of the two binning paths this view took (tests look at it)
        v.fused_result = None
        v.count_ready = None
        v.polled = False
        if v.fused:
            cap = v.spec_capacity
            up = lambda x: (x + 63) // 64 * 64          # 256-byte aligned slices of one int32 allocation
            o_keys_b, o_ord_a, o_ord_b, o_offs = 0, up(n), 2 * up(n), 3 * up(n)
            o_tk_a = 4 * up(n)
            o_tk_b, o_ix_a, o_ix_b = o_tk_a + up(cap), o_tk_a + 2 * up(cap), o_tk_a + 3 * up(cap)
            o_order = o_tk_a + 4 * up(cap)
            pool = torch.empty(o_order + up(v.num_tiles), dtype=i32, device=dev)
            base = pool.data_ptr()
            at = lambda off: C.c_void_p(base + 4 * off)
            v.total = torch.empty(1, dtype=torch.int64, device=dev)
            order_in_b, pairs_in_b = C.c_int(0), C.c_int(0)
            # tile ids that fit 16 bits travel through key expansion, pair sort and ranges as 16-bit keys
            narrow = bool(self.narrow_tile_keys and v.num_tiles <= (1 << 16))
            # Polling gains a few microseconds per view; a view whose binning takes milliseconds (hundreds of millions
            # of pairs) waits on an event instead, which costs it nothing by comparison and keeps the host thread free.
            v.polled = bool(self.poll_pair_count and n > 0 and cap <= POLL_MAX_PAIRS)
            if v.polled:
                v.slot.count_np[0] = _capi.COUNT_PENDING
            _capi.check(L.d3gs_bin_pairs(
                C.byref(v.Pd), _capi.ptr(v.radii), _capi.ptr(v.uvs), _capi.ptr(v.conic_opacity), _capi.ptr(v.depths),
                _capi.ptr(v.tiles_touched), _capi.ptr(v.tile_masks), _capi.ptr(v.depth_keys), at(o_keys_b), at(o_ord_a),
                at(o_ord_b), _capi.ptr(v.zero_ws_n), v.zero_ws_n.numel(), at(o_offs), _capi.ptr(v.zero_scan_ws),
                v.zero_scan_ws.numel(), _capi.ptr(v.total), C.c_void_p(v.slot.count_host.data_ptr()), cap, at(o_tk_a),
                at(o_tk_b), at(o_ix_a), at(o_ix_b), _capi.ptr(v.zero_ws_m), v.zero_ws_m.numel(), _capi.ptr(v.zero_ranges),
                at(o_order), _capi.BIN_WORKSPACES_ARE_ZERO | (_capi.BIN_HOST_COUNT_AT_END if v.polled else 0)
                | (_capi.BIN_KEYS_16BIT if narrow else 0),
                C.byref(order_in_b), C.byref(pairs_in_b), s), "d3gs_bin_pairs")
            if not v.polled:
                v.count_ready = torch.cuda.Event()
                v.count_ready.record()
            # what a second, exactly sized binning of this view would start from
            v.depth_keys_sorted = pool[o_keys_b:o_keys_b + n] if order_in_b.value else v.depth_keys
            v.gaussian_order = pool[o_ord_b:o_ord_b + n] if order_in_b.value else pool[o_ord_a:o_ord_a + n]
            v.counts_ordered = pool[o_offs:o_offs + n]
            o_tk, o_ix = (o_tk_b, o_ix_b) if pairs_in_b.value else (o_tk_a, o_ix_a)
            tile_keys = pool[o_tk:o_tk + cap].view(torch.int16)[:cap] if narrow else pool[o_tk:o_tk + cap]
            v.fused_result = (tile_keys, pool[o_ix:o_ix + cap], pool[o_order:o_order + v.num_tiles])
            return
        # The reference sorts all M pairs on the whole (tile, depth) key (render.py:845-887).  The depth
        # digits only depend on the gaussian, so the same stable order comes from sorting the N
        # gaussians by depth first, emitting the pairs in that order and sorting the pairs on the
        # tile digits only: 2 passes over M pairs instead of 6.
        with self._stage("depth_order"):
            v.depth_keys_sorted, v.gaussian_order = self._sort(
                v, v.depth_keys, torch.empty(n, dtype=i32, device=dev), n, 0, v.depth_bits, values_are_indices=True,
                zero_ws=v.zero_ws_n, status_slot=0)
        self._report_sort_status(v)
        with self._stage("scan"):
            # tile counts gathered into depth order and scanned in one launch
            v.counts_ordered = torch.empty(n, dtype=i32, device=dev)
            v.total = torch.empty(1, dtype=torch.int64, device=dev)
            _capi.check(L.d3gs_scan_gathered(_capi.ptr(v.tiles_touched), n, _capi.ptr(v.gaussian_order), n,
                                             _capi.ptr(v.counts_ordered), _capi.ptr(v.zero_scan_ws), v.zero_scan_ws.numel(), 1,
                                             _capi.ptr(v.total), C.c_void_p(v.slot.count_host.data_ptr()), s),
                        "d3gs_scan_gathered")
            # the scan also stores the count to pinned host memory; the host looks at it only after the
            # rest of the forward pass has been enqueued
            v.count_ready = torch.cuda.Event()
            v.count_ready.record()

    def _wait_pair_count(self, v) -> int:
        """The pair count of the view (or the negative status that replaces it), once it has reached the host."""
        if v.count_ready is not None:
            v.count_ready.synchronize()
        else:
            # the binning's last kernel stores the count (or a status) over the marker put there before the call
            arrived = poll_host_word(v.slot.count_np, _capi.COUNT_PENDING, POLL_SECONDS,
                                     torch.cuda.current_stream().synchronize)
            if arrived == "polled":
                v.slot.poll_timeouts = 0
            else:
                v.slot.poll_timeouts += 1
                if v.slot.poll_timeouts >= 3 and self.poll_pair_count:      # not one slow view: wait on an event from now on
                    self.poll_pair_count = False
                    warnings.warn("GaussianSplatOp: the pair count did not reach the host within "
                                  f"{POLL_SECONDS * 1e3:.0f} ms on three views in a row; polling is switched off "
                                  "for this operator (the host waits on an event instead)")
                if arrived == "never":
                    raise RuntimeError("d3gs_bin_pairs: the pair count never reached the host")
        return int(v.slot.count_host[0])

    # -- step 4: key expansion .. forward blend
    def _alloc_outputs(self, v):
        dev, batch, height, width = v.dev, v.batch, v.height, v.width
        f32, i32 = torch.float32, torch.int32
        v.final_T = torch.empty((batch, height, width), dtype=f32, device=dev)
        v.n_contrib = torch.empty((batch, height, width), dtype=i32, device=dev)
        channels = 4 if self._cfg.render_rgba else 3       # what the kernels write
        color_shape = (batch, channels, height, width) if self._cfg.use_nchw else (batch, height, width, channels)
        v.out_color = torch.empty(color_shape, dtype=f32, device=dev)
        v.out_depth = torch.empty((batch, height, width), dtype=f32, device=dev) if self._cfg.render_depth else None
        no_rgb = bool(self._cfg.disable_builtin_rgb)
        # disable_builtin_rgb: the caller's colour image is the alpha channel alone, or has no channel
        # (config_def.py:152-157)
        v.out = GaussianSplatOutput(custom_features=None, T=v.final_T, color=v.out_color[..., 3:] if no_rgb else v.out_color,
                                    depth=v.out_depth, n_contrib=v.n_contrib,
                                    radii=getattr(v, "radii", None) if v.n else torch.zeros(0, dtype=i32, device=dev),
                                    sparse_gaussian_ids=v.sparse_gaussian_ids, sparse_batch_ids=v.sparse_batch_ids)

    def _empty_result(self, v):
        """The render of a view without a single (tile, gaussian) pair.  The reference returns uninitialised buffers
        here (render.py:706-729); this fills in what an empty scene renders to."""
        out = v.out
        if v.custom_features is not None:
            out.custom_features = torch.zeros((v.batch, v.height, v.width, v.custom_features.shape[1]),
                                              dtype=torch.float32, device=v.dev)
        if getattr(v, "sh_done", None) is not None:
            torch.cuda.current_stream().wait_event(v.sh_done)
        v.final_T.fill_(1.0)
        v.n_contrib.zero_()
        v.out_color.zero_()
        if v.out_depth is not None:
            v.out_depth.zero_()
        if not v.training:
            bg = torch.tensor(np.asarray(self._cfg.bg_color, np.float32), device=v.dev).clamp(0, 1)
            if self._cfg.use_nchw:
                v.out_color[:, :3] = bg.view(1, 3, 1, 1)
            else:
                v.out_color[..., :3] = bg
        return out, None

    def _bin_and_blend(self, v, capacity: int, count_on_device: bool):
        """Key expansion .. blend for buffers of `capacity` pairs.  With count_on_device the kernels
        read the pair count from `total` on the device and nothing here waits for the host."""
        L, dev, s, Pd = self._lib, v.dev, v.s, v.Pd
        i32 = torch.int32
        if v.fused_result is not None and count_on_device:
            tile_keys_sorted, gaussian_idx_sorted, tile_order = v.fused_result
            workload_ranges = v.zero_ranges
            v.pooled_ranges_used = True
        else:
            m_dev = _capi.ptr(v.total) if count_on_device else None
            # pairs leave key expansion in depth order, so the pair sort only needs the tile id: 32-bit keys
            with self._stage("make_keys"):
                tile_keys = torch.empty(capacity, dtype=i32, device=dev)
                gaussian_idx = torch.empty(capacity, dtype=i32, device=dev)
                _capi.check(L.d3gs_make_keys(C.byref(Pd), _capi.ptr(v.radii), _capi.ptr(v.uvs), _capi.ptr(v.conic_opacity),
                                             _capi.ptr(v.depths), _capi.ptr(v.counts_ordered), _capi.ptr(v.gaussian_order),
                                             _capi.ptr(v.depth_keys_sorted), _capi.ptr(v.tile_masks), None,
                                             _capi.ptr(tile_keys), _capi.ptr(gaussian_idx), capacity, s),
                            "d3gs_make_keys")
            with self._stage("sort"):
                tile_keys_sorted, gaussian_idx_sorted = self._sort(
                    v, tile_keys, gaussian_idx, capacity, 0, v.tile_bits, m_dev,
                    zero_ws=v.zero_ws_m if count_on_device else None, status_slot=1)
            self._report_sort_status(v)
            v.pair_sort_done = torch.cuda.Event()
            v.pair_sort_done.record()
            with self._stage("tile_ranges"):
                # the pooled ranges serve the first binning of this view; a second one starts from fresh zeros
                workload_ranges = v.zero_ranges if not v.pooled_ranges_used else \
                    torch.zeros((v.num_tiles, 2), dtype=i32, device=dev)
                v.pooled_ranges_used = True
                tile_order = torch.empty(v.num_tiles, dtype=i32, device=dev)
                _capi.check(L.d3gs_tile_ranges_u32(_capi.ptr(tile_keys_sorted), capacity, m_dev,
                                                   _capi.ptr(workload_ranges), v.num_tiles, _capi.ptr(tile_order), s),
                            "d3gs_tile_ranges_u32")
        snap = None
        if v.training and self._cfg.rasterize_backward_algo == RasterizeBackwardAlgo.PER_GAUSSIAN:
            # K8 (render.py:940-962): where each tile's buckets start.  The bucket total stays on the device:
            # ceil(len / 64) summed over the tiles is at most pairs / 64 + tiles, which sizes the snapshots.
            bucket_offsets = torch.empty(v.num_tiles + 1, dtype=i32, device=dev)
            _capi.check(L.d3gs_bucket_offsets(_capi.ptr(workload_ranges), v.num_tiles, _capi.ptr(bucket_offsets), s),
                        "d3gs_bucket_offsets")
            max_buckets = capacity // _capi.BUCKET_SIZE + v.num_tiles + 1
            snap = (bucket_offsets, torch.empty((max_buckets, 256, self._snapshot_floats()), dtype=torch.float32, device=dev))
        ctx = GaussianSplatOpContext(
            conic_opacity=v.conic_opacity, radii=v.radii, uvs=v.uvs, rgb_gaussian=v.rgb_gaussian,
            gaussian_idx_sorted=gaussian_idx_sorted, workload_ranges=workload_ranges, per_gaussian_snap=snap,
            image_shape_wh=(v.width, v.height), cov2d_vecs=v.cov2d_vecs, sh_to_rgb_ne_0=v.ne0, depths=v.depths,
            tile_order=tile_order, grad_records=v.grad_records, grad_pool=v.grad_pool, grad_clear=v.grad_clear,
            grad_touched=v.grad_touched,
            kernel_color=v.out_color if v.no_rgb else None, instance_cameras=v.inst_cams, instance_ids=v.inst_ids,
            batch_size=v.batch, batch_cameras=v.batch_cams, sparse_gaussian_ids=v.sparse_gaussian_ids,
            sparse_batch_ids=v.sparse_batch_ids if (v.sparse and v.batch > 1) else None)
        # The view's kernel parameters, for a backward pass over the same model and cameras.  The model and the
        # cameras are remembered weakly and by what the parameters depend on: backward() rebuilds the parameters
        # when it is handed other objects, or the same ones changed in place where that can be seen.
        ctx._forward_params = (_capi.Params.from_buffer_copy(v.P), weakref.ref(v.model), weakref.ref(v.cameras),
                               bool(v.training), self._params_signature(v.model, v.cameras))
        if v.sh_done is not None:
            v.main_stream.wait_event(v.sh_done)      # (the stream object of the fork: forward runs on one stream)
        with self._stage("blend_fwd"):
            self.rasterize_forward_backward(v.model, ctx, v.out, training=v.training,
                                            render_depth=self._cfg.render_depth, _params=Pd)
        return ctx, tile_keys_sorted

    def _bundle_in_one_pass(self, batch, cameras) -> bool:
        """A bundle of B cameras goes through the kernels in ONE pass over B * N render items, as the reference's
        does (render.py:314-326, 787, 809, 1515-1522), unless it uses an option whose host code here is written
        per camera (the fused single-stream preprocess), or the 32-bit sort when the bundle's tiles
        outgrow its 14 tile bits (the reference asserts there, render.py:227-228).  Those bundles are rendered camera
        by camera (_forward_bundle)."""
        c = self._cfg
        if not (self.bundle_in_one_pass and batch > 1 and (self.overlap_sh_colors or c.sparse_mode)):
            return False
        if c.enable_32bit_sort:
            width, height = cameras.image_shape_wh
            return batch * div_up(width, 16) * div_up(height, 16) < 2 ** 14
        return True

    def _forward_bundle(self, model, cameras: "CameraBundle", training, instance2world_T, custom_features, mask,
                        prep_user_inputs):
        """A bundle of B cameras rendered as B single-camera passes over the shared model (the fallback for the
        options _bundle_in_one_pass lists).  Outputs are stacked along the batch axis; radii and the mask
        are flat [B * N] as in the reference."""
        B, n = len(cameras), len(model)
        assert B > 0, "empty camera bundle"
        if mask is not None:
            assert mask.numel() == B * n, "mask must have one entry per (camera, gaussian)"
            mask = mask.reshape(B, n)
        if custom_features is not None:      # one row per (camera, gaussian) (render.py:245)
            assert custom_features.ndim == 2 and custom_features.shape[0] == B * n, "custom_features must be [B * N, F]"
        outs, ctxs, cams, rendered = [], [], [], 0
        for b in range(B):
            cam_b = cameras.select(b)
            out_b, ctx_b = self.forward(model, cam_b, training, instance2world_T,
                                        None if custom_features is None else custom_features[b * n:(b + 1) * n],
                                        None if mask is None else mask[b].contiguous(), prep_user_inputs)
            outs.append(out_b)
            ctxs.append(ctx_b)
            cams.append(cam_b)
            rendered += self.last_num_rendered
        self.last_num_rendered = rendered
        cat = lambda name: torch.cat([getattr(o, name) for o in outs], 0)
        out = GaussianSplatOutput(custom_features=cat("custom_features") if custom_features is not None else None,
                                  T=cat("T"), color=cat("color"),
                                  depth=cat("depth") if outs[0].depth is not None else None,
                                  n_contrib=cat("n_contrib"), radii=cat("radii"))
        if self._cfg.sparse_mode:       # rows of camera 0, then camera 1, ... (render.py:494: sparse_batch_id)
            out.sparse_gaussian_ids = cat("sparse_gaussian_ids")
            out.sparse_batch_ids = torch.cat([torch.full_like(o.sparse_gaussian_ids, b) for b, o in enumerate(outs)], 0)
        if not training:
            return out, None
        rows = [int(o.sparse_gaussian_ids.numel()) for o in outs] if self._cfg.sparse_mode else None
        return out, GaussianSplatOpBatchContext(per_camera=ctxs, cameras=cams, image_shape_wh=cameras.image_shape_wh,
                                                rows_per_camera=rows)

    # ------------------------------------------------------- sparse bundles: K10
    def unique_ids(self, ids: torch.Tensor, id_limit: int):
        """Distinct values of ``ids`` (int32 [R], each in [0, id_limit)) in ascending order, and the rows grouped by
        value: ``(unique [U], run_rows [R], run_starts [R + 1])`` (render.py:2864-2903 does this with a hash table).
        One host synchronisation: U sizes the result."""
        assert ids.is_cuda and ids.dtype == torch.int32 and ids.ndim == 1 and ids.is_contiguous()
        L, s, dev, R = self._lib, self._stream(), ids.device, int(ids.numel())
        i32 = torch.int32
        nbytes = C.c_size_t(0)
        _capi.check(L.d3gs_unique_ids_workspace_bytes(R, int(id_limit), C.byref(nbytes)), "d3gs_unique_ids_workspace_bytes")
        ws = torch.empty(max(nbytes.value, 1), dtype=torch.uint8, device=dev)
        unique = torch.empty(R, dtype=i32, device=dev)
        inverse, run_rows = torch.empty(R, dtype=i32, device=dev), torch.empty(R, dtype=i32, device=dev)
        run_starts = torch.empty(R + 1, dtype=i32, device=dev)
        count_dev = torch.empty(1, dtype=torch.int64, device=dev)
        slot = self._slot(dev)
        _capi.check(L.d3gs_unique_ids(_capi.ptr(ids), R, int(id_limit), _capi.ptr(unique), _capi.ptr(inverse),
                                      _capi.ptr(run_rows), _capi.ptr(run_starts), _capi.ptr(ws), nbytes.value,
                                      _capi.ptr(count_dev), C.c_void_p(slot.count_host.data_ptr()), s), "d3gs_unique_ids")
        torch.cuda.current_stream().synchronize()
        U = int(slot.count_host[0])
        if U < 0:
            raise RuntimeError("d3gs_unique_ids: a workgroup's bounded wait on an earlier chunk ran out")
        self.last_unique_inverse = inverse
        return unique[:U], run_rows, run_starts

    def merge_rows(self, rows: torch.Tensor, run_rows: torch.Tensor, run_starts: torch.Tensor, n_runs: int):
        """``merged[u] = sum of rows[r]`` over the rows r of run u (see ``unique_ids``), in run order."""
        rows = rows.contiguous()
        R = int(rows.shape[0])
        width = int(rows.numel() // max(R, 1))
        merged = torch.empty((n_runs,) + tuple(rows.shape[1:]), dtype=torch.float32, device=rows.device)
        _capi.check(self._lib.d3gs_merge_rows(_capi.ptr(rows), R, width, _capi.ptr(run_rows), _capi.ptr(run_starts),
                                              int(n_runs), _capi.ptr(merged), self._stream()), "d3gs_merge_rows")
        return merged

    def _backward_bundle(self, model, ctx, out, grad, return_uv_grad, instance2world_T=None):
        return _backward_bundle_impl(self, model, ctx, out, grad, return_uv_grad, instance2world_T)

    # ------------------------------------------------------- gradient pool
    @staticmethod
    def _grad_fields(model, rows=None):
        """(name, shape) of the gradient arrays: the model's own shapes, or `rows` rows of them (sparse mode)."""
        fields = [("xyz", model.xyz), ("quaternion_xyzw", model.quaternion_xyzw), ("scale", model.scale),
                  ("opacity", model.opacity), ("color_sh", model.color_sh)]
        if model.color_sh_base is not None:
            fields.append(("color_sh_base", model.color_sh_base))
        return [(name, tuple(t.shape) if rows is None else (rows,) + tuple(t.shape[1:])) for name, t in fields]

    @classmethod
    def _grad_pool_floats(cls, model, rows=None) -> int:
        return sum((math.prod(shape) + 63) // 64 * 64 for _, shape in cls._grad_fields(model, rows))

    @classmethod
    def _grad_views(cls, model, pool, rows=None):
        """The model-shaped gradient tensors as 256-byte aligned slices of one allocation."""
        views, off = {}, 0
        for name, shape in cls._grad_fields(model, rows):
            numel = math.prod(shape)
            views[name] = pool[off:off + numel].view(shape)
            off += (numel + 63) // 64 * 64
        return views

    # ------------------------------------------------------- custom features
    # The blend is linear in the per-gaussian channel values and every channel shares the weights
    # alpha * T, so F custom feature channels (render.py:1536-1539, 1892-1923, 1952-1971) are blended by
    # running the colour kernels again over three channels at a time; in the backward pass each such
    # run adds its share of d(uv, conic, opacity) and yields the gradient of its three channels where a
    # colour run yields dcolor.
    @staticmethod
    def _feature_params(P: _capi.Params) -> _capi.Params:
        Q = _capi.Params.from_buffer_copy(P)
        Q.training, Q.render_depth, Q.render_rgba, Q.use_nchw = 1, 0, 0, 0     # raw sums, [H, W, 3]
        return Q

    @staticmethod
    def _feature_triples(feat: torch.Tensor):
        n, F = feat.shape
        for k in range(0, F, 3):
            tri = torch.zeros((n, 3), dtype=torch.float32, device=feat.device)
            tri[:, :min(3, F - k)] = feat[:, k:k + 3]
            yield k, min(3, F - k), tri

    def _blend_custom_features(self, P, ctx, out, feat):
        """The feature image [B, H, W, F]: the library's feature kernels (up to 16 channels beside one evaluation of
        alpha), or with ``feature_kernels`` off three channels at a time through the colour kernel."""
        L, s = self._lib, self._stream()
        Q = self._feature_params(P)
        B, H, W = out.T.shape        # a bundle in one pass: B images, feature rows of the B * N render items
        res = torch.empty((B, H, W, feat.shape[1]), dtype=torch.float32, device=feat.device)
        if self.feature_kernels:
            _capi.check(L.d3gs_blend_features_fwd(
                C.byref(Q), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(feat.detach()), int(feat.shape[1]), _capi.ptr(ctx.tile_order),
                _capi.ptr(res), s), "d3gs_blend_features_fwd")
            return res
        T2, nc2 = torch.empty_like(out.T), torch.empty_like(out.n_contrib)
        for k, w, tri in self._feature_triples(feat.detach()):
            img = torch.empty((B, H, W, 3), dtype=torch.float32, device=feat.device)
            _capi.check(L.d3gs_blend_fwd(
                C.byref(Q), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(tri), None, _capi.ptr(ctx.tile_order), _capi.ptr(img),
                _capi.ptr(T2), _capi.ptr(nc2), None, None, 0, s), "d3gs_blend_fwd (custom features)")
            res[..., k:k + w] = img[..., :w]
        return res

    def _backward_custom_features(self, P, ctx, out, dfeat_img, rec, touched=None):
        """Adds the feature channels' share to rec[:, 0:6] and returns dcustom_features, one row per render item
        like the features; gaussians that receive anything are marked in ``touched`` as in the colour pass."""
        L, s = self._lib, self._stream()
        Q = self._feature_params(P)
        feat = ctx.custom_features.detach()
        n, F = feat.shape
        B, H, W = out.T.shape
        if self.feature_kernels:
            dfeat = torch.zeros((n, F), dtype=torch.float32, device=feat.device)
            _capi.check(L.d3gs_blend_features_bwd(
                C.byref(Q), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(feat), int(F), _capi.ptr(ctx.tile_order),
                _capi.ptr(out.n_contrib), _capi.ptr(out.custom_features.detach().contiguous()), _capi.ptr(dfeat_img),
                _capi.ptr(rec), _capi.ptr(dfeat), _capi.ptr(touched), s), "d3gs_blend_features_bwd")
            return dfeat
        dfeat = torch.empty((n, F), dtype=torch.float32, device=feat.device)
        zero_dT = torch.zeros_like(out.T)
        for k, w, tri in self._feature_triples(feat):
            img = torch.zeros((B, H, W, 3), dtype=torch.float32, device=feat.device)
            img[..., :w] = out.custom_features[..., k:k + w]
            dimg = torch.zeros((B, H, W, 3), dtype=torch.float32, device=feat.device)
            dimg[..., :w] = dfeat_img[..., k:k + w]
            rec_k = torch.zeros_like(rec)
            _capi.check(L.d3gs_blend_bwd(
                C.byref(Q), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(tri), None, _capi.ptr(ctx.tile_order), _capi.ptr(out.T),
                _capi.ptr(out.n_contrib), _capi.ptr(img), None, _capi.ptr(dimg), _capi.ptr(zero_dT), None,
                _capi.ptr(rec_k), _capi.ptr(touched), s), "d3gs_blend_bwd (custom features)")
            rec[:, 0:6] += rec_k[:, 0:6]
            dfeat[:, k:k + w] = rec_k[:, 6:6 + w]
        return dfeat

    # ------------------------------------------------------- blend fwd / bwd
    def rasterize_forward_backward(self, model, ctx: GaussianSplatOpContext, out: GaussianSplatOutput,
                                   grad: GaussianSplatGradients | None = None, training: bool = False,
                                   render_depth: bool = False, custom_features=None, _params=None, _cameras=None):
        """render.py:1329-2316: blend forward when ``grad`` is None, else blend backward."""
        assert bool(render_depth) == bool(self._cfg.render_depth), "render_depth must match the op's config"
        L = self._lib
        P = _params
        if P is None:
            assert _cameras is not None, "camera needed to rebuild kernel parameters"
            P = self.make_params(model, _cameras, training)
        s = self._stream()
        n, dev = int(ctx.radii.numel()), ctx.uvs.device      # render items (sparse mode: the accepted ones)
        color = ctx.kernel_color if ctx.kernel_color is not None else out.color
        if grad is None:
            clear, ctx.grad_clear = ctx.grad_clear, None
            if ctx.per_gaussian_snap is not None:      # the forward also stores the pixels' state per bucket
                bucket_offsets, snapshots = ctx.per_gaussian_snap
                _capi.check(L.d3gs_blend_fwd_snapshots(
                    C.byref(P), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                    _capi.ptr(ctx.conic_opacity), _capi.ptr(ctx.rgb_gaussian), _capi.ptr(ctx.depths),
                    _capi.ptr(ctx.tile_order), _capi.ptr(color), _capi.ptr(out.T), _capi.ptr(out.n_contrib),
                    _capi.ptr(out.depth), _capi.ptr(clear), 0 if clear is None else clear.numel() * 4,
                    _capi.ptr(bucket_offsets), _capi.ptr(snapshots), s), "d3gs_blend_fwd_snapshots")
                return None
            _capi.check(L.d3gs_blend_fwd(
                C.byref(P), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(ctx.rgb_gaussian), _capi.ptr(ctx.depths),
                _capi.ptr(ctx.tile_order), _capi.ptr(color), _capi.ptr(out.T), _capi.ptr(out.n_contrib),
                _capi.ptr(out.depth), _capi.ptr(clear), 0 if clear is None else clear.numel() * 4, s), "d3gs_blend_fwd")
            return None
        drgb = grad.drgb
        assert drgb.shape == out.color.shape, "drgb must have the shape of the colour image"
        if ctx.kernel_color is not None:      # gradient of the alpha channel only; the colour channels carry none
            full = torch.zeros_like(color)
            full[..., 3:] = drgb
            drgb = full
        assert drgb.is_contiguous(), "drgb must be contiguous"
        assert grad.dT.is_contiguous(), "dT must be contiguous"
        ddepth = None
        if render_depth:
            ddepth = grad.ddepth if grad.ddepth is not None else torch.zeros_like(out.depth)
            assert ddepth.is_contiguous() and ddepth.shape == out.depth.shape, "ddepth must be contiguous [1,H,W]"
        # one 64-byte record per gaussian (see D3GS_GRAD_RECORD_FLOATS); the reference's four tensors
        # and dz are strided views of it
        rec, ctx.grad_records = ctx.grad_records, None
        touched, ctx.grad_touched = ctx.grad_touched, None
        counter = None
        if self._cfg.measure_atomic_add_count:     # config_def.py:134; render.py:2310-2311
            counter = torch.zeros(1, dtype=torch.int32, device=dev)
            P = _capi.Params.from_buffer_copy(P)
            P.atomic_add_count = counter.data_ptr()
        if rec is None:     # a second backward over this context: fresh records, work found from the records
            rec = torch.zeros((n, _capi.GRAD_RECORD_FLOATS), dtype=torch.float32, device=dev)
            touched = None
        if ctx.per_gaussian_snap is not None:      # rasterize_backward_algo = PER_GAUSSIAN (render.py:2319-2776)
            bucket_offsets, snapshots = ctx.per_gaussian_snap
            _capi.check(L.d3gs_blend_bwd_per_gaussian(
                C.byref(P), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(ctx.rgb_gaussian), _capi.ptr(ctx.depths),
                _capi.ptr(ctx.tile_order), _capi.ptr(out.T), _capi.ptr(out.n_contrib), _capi.ptr(color),
                _capi.ptr(out.depth), _capi.ptr(drgb), _capi.ptr(grad.dT), _capi.ptr(ddepth),
                _capi.ptr(bucket_offsets), _capi.ptr(snapshots), _capi.ptr(rec), _capi.ptr(touched), s),
                "d3gs_blend_bwd_per_gaussian")
        else:
            _capi.check(L.d3gs_blend_bwd(
                C.byref(P), _capi.ptr(ctx.workload_ranges), _capi.ptr(ctx.gaussian_idx_sorted), _capi.ptr(ctx.uvs),
                _capi.ptr(ctx.conic_opacity), _capi.ptr(ctx.rgb_gaussian), _capi.ptr(ctx.depths),
                _capi.ptr(ctx.tile_order), _capi.ptr(out.T), _capi.ptr(out.n_contrib), _capi.ptr(color),
                _capi.ptr(out.depth), _capi.ptr(drgb), _capi.ptr(grad.dT), _capi.ptr(ddepth), _capi.ptr(rec),
                _capi.ptr(touched), s), "d3gs_blend_bwd")
        if counter is not None:
            # global atomic requests of this blend backward (one per (tile, gaussian) with a non-zero sum); the
            # reference prints its count the same way
            self.last_atomic_add_count = int(counter.item())
            if self._cfg.verbose:
                print(f"atomic add count: {self.last_atomic_add_count}")
        res = RasterizeGradientOutput(duv=rec[:, 0:2], dconic=rec[:, 2:5], dopacity=rec[:, 5], dcolor=rec[:, 6:9],
                                      dz=rec[:, 9] if render_depth else None, records=rec, touched=touched)
        return res

    # --------------------------------------------------------------- backward
    def backward(self, model: GaussianModelOriginBase, cameras, ctx: GaussianSplatOpContext, out: GaussianSplatOutput,
                 grad: GaussianSplatGradients, return_uv_grad: bool = False, instance2world_T=None,
                 custom_features=None, prep_user_inputs=None):
        """render.py:2779-3374.  Returns ``(grad_model, duv | None, dcustom_features)``; ``grad_model``
        is a model-shaped dataclass holding the gradients of the raw tensors."""
        if prep_user_inputs:
            raise NotImplementedError("prep_user_inputs is not supported")
        if isinstance(ctx, GaussianSplatOpBatchContext):
            return self._backward_bundle(model, ctx, out, grad, return_uv_grad, instance2world_T)
        L = self._lib
        kept = getattr(ctx, "_forward_params", None)
        if kept is not None and kept[1]() is model and kept[2]() is cameras and kept[3] \
                and kept[4] == self._params_signature(model, cameras):
            P = _capi.Params.from_buffer_copy(kept[0])      # (a copy: sparse mode edits n below)
        else:
            P = self.make_params(model, cameras, True, ctx.batch_cameras)
        s = self._stream()
        sparse_ids = ctx.sparse_gaussian_ids
        B = ctx.batch_size
        if sparse_ids is not None:      # the kernels see a scene of the V accepted gaussians
            P.n = int(sparse_ids.numel())
            if B > 1:                   # ... of a bundle: compact rows, each with the camera sparse_batch_ids names
                P.compact_items = P.n
        n, dev = P.n, model.xyz.device
        with self._stage("blend_bwd"):
            g = self.rasterize_forward_backward(model, ctx, out, grad, training=True,
                                                render_depth=self._cfg.render_depth, _params=P)
        dcustom = None
        if ctx.custom_features is not None:
            dfeat_img = grad.dcustom_features if grad.dcustom_features is not None else \
                torch.zeros_like(out.custom_features)
            dcustom = self._backward_custom_features(P, ctx, out, dfeat_img.contiguous(), g.records, g.touched)
        with self._stage("preprocess_bwd"):
            pool, ctx.grad_pool = ctx.grad_pool, None
            grad_rows = None if sparse_ids is None else n     # sparse mode: one gradient row per accepted gaussian
            prezeroed = pool is not None and pool.numel() == self._grad_pool_floats(model, grad_rows)
            if not prezeroed:
                pool = torch.empty(self._grad_pool_floats(model, grad_rows), dtype=torch.float32, device=dev)
            gv = self._grad_views(model, pool, grad_rows)
            dxyz, dquat, dscale, dopacity, dsh = (gv[k] for k in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh"))
            dsh_base = gv.get("color_sh_base")
            # the cameras of the forward pass; a context from a pass without instances takes the argument
            inst_ids, inst_cams = ctx.instance_ids, ctx.instance_cameras
            if inst_cams is None and instance2world_T is not None:
                inst_ids, inst_cams = self.instance_table(model, cameras, instance2world_T)
            # The reference loops over the batch inside its kernel (render.py:2972-2989), and so does the library's;
            # with bundle_k9_in_one_launch off, one launch per camera instead: camera b works on its own rows of the
            # per-item arrays, the first call stores, the others add.
            if sparse_ids is not None:
                # sparse gradient (render.py:2918, 3185-3213): row i belongs to gaussian sparse_gaussian_ids[i]
                _capi.check(L.d3gs_preprocess_bwd_sparse(
                    C.byref(P), _capi.ptr(sparse_ids), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw),
                    _capi.ptr(model.scale), _capi.ptr(model.opacity), _capi.ptr(model.color_sh), _capi.ptr(ctx.radii),
                    _capi.ptr(ctx.cov2d_vecs), _capi.ptr(ctx.sh_to_rgb_ne_0), _capi.ptr(g.records), _capi.ptr(g.touched),
                    int(self._cfg.compat_ref_sh_mask_bitorder), int(prezeroed), _capi.ptr(dxyz), _capi.ptr(dquat),
                    _capi.ptr(dscale), _capi.ptr(dopacity), _capi.ptr(dsh), _capi.ptr(dsh_base),
                    self._instances_arg(inst_ids, inst_cams, B), _capi.ptr(ctx.sparse_batch_ids), s),
                    "d3gs_preprocess_bwd_sparse")
            if sparse_ids is None and (B == 1 or self.bundle_k9_in_one_launch):
                # dense: one launch, which for a bundle works every gaussian off camera after camera
                _capi.check(L.d3gs_preprocess_bwd(
                    C.byref(P), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw),
                    _capi.ptr(model.scale), _capi.ptr(model.opacity), _capi.ptr(model.color_sh),
                    _capi.ptr(ctx.radii), _capi.ptr(ctx.cov2d_vecs), _capi.ptr(ctx.sh_to_rgb_ne_0), _capi.ptr(g.records),
                    _capi.ptr(g.touched), int(self._cfg.compat_ref_sh_mask_bitorder), int(prezeroed), _capi.ptr(dxyz),
                    _capi.ptr(dquat), _capi.ptr(dscale), _capi.ptr(dopacity), _capi.ptr(dsh), _capi.ptr(dsh_base),
                    self._instances_arg(inst_ids, inst_cams, B), s), "d3gs_preprocess_bwd")
            rows = lambda t, b: None if t is None else t[b * n:(b + 1) * n]
            for b in range(B if (sparse_ids is None and B > 1 and not self.bundle_k9_in_one_launch) else 0):
                inst = self._instances_arg(inst_ids, inst_cams, B, b)      # the instance poses as camera b sees them
                _capi.check(L.d3gs_preprocess_bwd_camera(
                    C.byref(P), b, int(b > 0), _capi.ptr(model.xyz), _capi.ptr(model.quaternion_xyzw),
                    _capi.ptr(model.scale), _capi.ptr(model.opacity), _capi.ptr(model.color_sh),
                    _capi.ptr(rows(ctx.radii, b)), _capi.ptr(rows(ctx.cov2d_vecs, b)),
                    _capi.ptr(rows(ctx.sh_to_rgb_ne_0, b)), _capi.ptr(rows(g.records, b)), _capi.ptr(rows(g.touched, b)),
                    int(self._cfg.compat_ref_sh_mask_bitorder), int(prezeroed), _capi.ptr(dxyz), _capi.ptr(dquat),
                    _capi.ptr(dscale), _capi.ptr(dopacity), _capi.ptr(dsh), _capi.ptr(dsh_base), inst, s),
                    "d3gs_preprocess_bwd")
        grad_model = dataclasses.replace(model, xyz=dxyz, quaternion_xyzw=dquat, scale=dscale, opacity=dopacity,
                                         color_sh=dsh, color_sh_base=dsh_base)
        self.last_raster_grads = g
        if sparse_ids is not None and B > 1:
            # A sparse bundle in one pass: one row per accepted (camera, gaussian); the rows of a gaussian that
            # several cameras accepted are merged (render.py:2864-2903) into one row per distinct gaussian, ascending
            unique, run_rows, run_starts = self.unique_ids(sparse_ids, len(model))
            self.last_sparse_unique_ids = unique
            merged = {name: self.merge_rows(getattr(grad_model, name), run_rows, run_starts, int(unique.numel()))
                      for name in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh", "color_sh_base")
                      if getattr(grad_model, name) is not None}
            grad_model = dataclasses.replace(model, **merged)
            # duv keeps one row per accepted (camera, gaussian), cameras one after the other, as out.sparse_gaussian_ids
            return grad_model, (g.duv.reshape(1, n, 2) if return_uv_grad else None), dcustom
        if return_uv_grad:
            return grad_model, g.duv.reshape(B, n, 2), dcustom
        return grad_model, None, dcustom


def _backward_bundle_sparse(op, model, ctx, out, grad, return_uv_grad, instance2world_T=None):
    """Sparse-mode bundle (render.py:2864-2903): each camera has its own accepted gaussians; the gradient rows of a
    gaussian seen by several cameras are merged.  The reference deduplicates the ids with a hash table
    (insert, collect, query); here the library sorts them and numbers the runs of equal ids (d3gs_unique_ids), which
    also fixes the row order: the result has one row per distinct accepted gaussian, ascending, and
    ``op.last_sparse_unique_ids`` names them; d3gs_merge_rows adds each gaussian's rows in camera order."""
    parts, duvs, offs = [], [], 0
    dev = model.xyz.device
    for b, (ctx_b, cam_b) in enumerate(zip(ctx.per_camera, ctx.cameras)):
        # the camera's rows of out.radii / out.sparse_gaussian_ids: it has them even when its accepted gaussians ended
        # without a single (tile, gaussian) pair, in which case there is no context and its gradients are zero
        v = ctx.rows_per_camera[b] if ctx.rows_per_camera is not None else \
            (0 if ctx_b is None else int(ctx_b.sparse_gaussian_ids.numel()))
        sl = slice(offs, offs + v)
        offs += v
        if ctx_b is None:
            duvs.append(torch.zeros((v, 2), dtype=torch.float32, device=dev))
            continue
        g_b = GaussianSplatGradients(drgb=grad.drgb[b:b + 1].contiguous(), dT=grad.dT[b:b + 1].contiguous(),
                                     ddepth=None if grad.ddepth is None else grad.ddepth[b:b + 1].contiguous())
        out_b = out.select_batch(b)
        out_b.radii = out.radii[sl]
        gm, duv, _ = op.backward(model, cam_b, ctx_b, out_b, g_b, return_uv_grad=True, instance2world_T=instance2world_T)
        parts.append((ctx_b.sparse_gaussian_ids, gm))
        duvs.append(duv[0])
    if not parts:
        op.last_sparse_unique_ids = torch.zeros(0, dtype=torch.int32, device=dev)
        zeros = {k: torch.zeros((0,) + tuple(v.shape[1:]), dtype=v.dtype, device=dev)
                 for k, v in model.get_proxy_field_dict().items()}
        return dataclasses.replace(model, **zeros), (torch.cat(duvs, 0).unsqueeze(0) if return_uv_grad and duvs else None), None
    all_ids = torch.cat([ids for ids, _ in parts], 0).to(torch.int32).contiguous()
    unique, run_rows, run_starts = op.unique_ids(all_ids, len(model))
    op.last_sparse_unique_ids = unique
    merged = {}
    for name in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh", "color_sh_base"):
        if getattr(model, name) is None:
            continue
        rows = torch.cat([getattr(gm, name) for _, gm in parts], 0)
        merged[name] = op.merge_rows(rows, run_rows, run_starts, int(unique.numel()))
    # duv: one row per accepted (camera, gaussian), cameras one after the other, as out.sparse_gaussian_ids
    return dataclasses.replace(model, **merged), (torch.cat(duvs, 0).unsqueeze(0) if return_uv_grad else None), None


def _backward_bundle_impl(op, model, ctx, out, grad, return_uv_grad, instance2world_T=None):
    """Per-camera backward passes; the model gradients add up over the cameras, duv stays per camera."""
    if op._cfg.sparse_mode:
        return _backward_bundle_sparse(op, model, ctx, out, grad, return_uv_grad, instance2world_T)
    total, duvs, dcfs = None, [], []
    n = len(model)
    for b, (ctx_b, cam_b) in enumerate(zip(ctx.per_camera, ctx.cameras)):
        if ctx_b is None:       # nothing was rendered for this camera: zero gradient
            duvs.append(torch.zeros((1, n, 2), dtype=torch.float32, device=model.xyz.device))
            if out.custom_features is not None:
                dcfs.append(torch.zeros((n, out.custom_features.shape[-1]), dtype=torch.float32, device=model.xyz.device))
            continue
        g_b = GaussianSplatGradients(
            drgb=grad.drgb[b:b + 1].contiguous(), dT=grad.dT[b:b + 1].contiguous(),
            ddepth=None if grad.ddepth is None else grad.ddepth[b:b + 1].contiguous(),
            dcustom_features=None if grad.dcustom_features is None else grad.dcustom_features[b:b + 1].contiguous())
        gm, duv, dcf = op.backward(model, cam_b, ctx_b, out.select_batch(b), g_b, return_uv_grad=True,
                                   instance2world_T=instance2world_T)
        duvs.append(duv)
        if dcf is not None:
            dcfs.append(dcf)
        if total is None:
            total = gm
        else:
            for name in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh", "color_sh_base"):
                t = getattr(total, name)
                if t is not None:
                    t.add_(getattr(gm, name))
    if total is None:
        zeros = {k: torch.zeros_like(v) for k, v in model.get_proxy_field_dict().items()}
        total = dataclasses.replace(model, **zeros)
    # feature gradients: rows of camera 0, then camera 1, ..., like the features themselves
    return total, (torch.cat(duvs, 0) if return_uv_grad else None), (torch.cat(dcfs, 0) if dcfs else None)


class _RasterizeGaussians(torch.autograd.Function):
    """render.py:3376-3587, with saved tensors addressed by name."""

    @staticmethod
    def forward(ctx, xyz, color_sh, color_sh_base, scale, quaternion_xyzw, opacity, cur_sh_degree, custom_features,
                mask, model_cls, cameras, training, op: GaussianSplatOp, uv_grad_holder=None, instance_id=None,
                instance2world_T=None):
        model = model_cls(xyz=xyz, color_sh=color_sh, color_sh_base=color_sh_base, scale=scale,
                          quaternion_xyzw=quaternion_xyzw, opacity=opacity, cur_sh_degree=cur_sh_degree,
                          instance_id=instance_id, act_applied=True)
        out, fwd_ctx = op.forward(model, cameras, training, instance2world_T, custom_features=custom_features,
                                  mask=mask)
        ctx.has_ctx = fwd_ctx is not None
        if fwd_ctx is not None:
            ctx.fwd_ctx = fwd_ctx
            ctx.out = out
        ctx.model = model
        ctx.op = op
        ctx.cameras = cameras
        ctx.return_uv_grad = uv_grad_holder is not None
        ctx.mark_non_differentiable(out.n_contrib, out.radii)
        # same tuple as the reference (render.py:3493-3499)
        return out.color, out.depth, out.custom_features, out.T, out.n_contrib, out.radii

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, drgb, ddepth, dcustom_features, dT, dn_contrib, dradii):
        if not ctx.has_ctx:
            return (None,) * 16
        if drgb is None:
            drgb = torch.zeros_like(ctx.out.color)
        if dT is None:
            dT = torch.zeros_like(ctx.out.T)
        if ddepth is not None:
            ddepth = ddepth.contiguous()
        if dcustom_features is not None:
            dcustom_features = dcustom_features.contiguous()
        grads = GaussianSplatGradients(drgb=drgb.contiguous(), dT=dT.contiguous(), ddepth=ddepth,
                                       dcustom_features=dcustom_features)
        gm, duv, dcf = ctx.op.backward(ctx.model, ctx.cameras, ctx.fwd_ctx, ctx.out, grads,
                                       return_uv_grad=ctx.return_uv_grad)
        # no gradient reaches the instance poses (render.py:3584-3587 returns None for them as well)
        return (gm.xyz, gm.color_sh, gm.color_sh_base, gm.scale, gm.quaternion_xyzw, gm.opacity, None, dcf, None,
                None, None, None, None, duv, None, None)


def rasterize_gaussians(model: GaussianModelOriginBase, cameras, op: GaussianSplatOp, training=False,
                        uv_grad_holder: torch.Tensor | None = None, instance2world_T=None, custom_features=None,
                        mask=None) -> GaussianSplatOutput:
    """render.py:3783-3838."""
    model = model.create_model_with_act()   # torch-side activations for the non-fused families
    res = _RasterizeGaussians.apply(model.xyz, model.color_sh, model.color_sh_base, model.scale,
                                    model.quaternion_xyzw, model.opacity, model.cur_sh_degree, custom_features, mask,
                                    type(model), cameras, training, op, uv_grad_holder, model.instance_id,
                                    instance2world_T)
    return GaussianSplatOutput(color=res[0], depth=res[1], custom_features=res[2], T=res[3], n_contrib=res[4],
                               radii=res[5])


def __getattr__(name):
    # render.py:3840-3891 lives beside rasterize_gaussians in the reference; here it is defined with the
    # time-dependent model family it serves (pvg.py imports this module, hence the late lookup)
    if name == "rasterize_gaussians_dynamic":
        from .pvg import rasterize_gaussians_dynamic
        return rasterize_gaussians_dynamic
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
