"""Minimal camera carriers with the attributes the rasterizer reads.

Stand-ins for the reference's ``BasicPinholeCamera`` (d3sim/data/scene_def/camera.py:55-61,
184-190) and ``Pose`` (d3sim/data/scene_def/base.py:138-140): ``intrinsic`` 4x4,
``pose.to_world`` 4x4 (camera -> world), ``image_shape_wh``, ``frame_local_id``,
``focal_length``, ``principal_point``.
"""
from __future__ import annotations

import dataclasses

import numpy as np


@dataclasses.dataclass
class Pose:
    to_world: np.ndarray = dataclasses.field(default_factory=lambda: np.eye(4))


@dataclasses.dataclass
class BasicPinholeCamera:
    intrinsic: np.ndarray
    image_shape_wh: tuple[int, int]
    pose: Pose = dataclasses.field(default_factory=Pose)
    frame_local_id: int | None = None

    @property
    def focal_length(self) -> np.ndarray:
        return np.array([self.intrinsic[0, 0], self.intrinsic[1, 1]])

    @property
    def principal_point(self) -> np.ndarray:
        return np.array([self.intrinsic[0, 2], self.intrinsic[1, 2]])

    @classmethod
    def from_params(cls, fx, fy, cx, cy, width, height, to_world=None):
        K = np.eye(4, dtype=np.float64)
        K[0, 0], K[1, 1], K[0, 2], K[1, 2] = fx, fy, cx, cy
        pose = Pose(np.eye(4) if to_world is None else np.asarray(to_world, np.float64))
        return cls(intrinsic=K, image_shape_wh=(int(width), int(height)), pose=pose)
