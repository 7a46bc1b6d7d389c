"""
Compute devices, mirroring heat/core/devices.py:17-207: ``ht.cpu``, ``ht.gpu`` (registered only when
a GPU is visible, as ``cuda:{rank % device_count}``), ``get_device``, ``sanitize_device``,
``use_device``.
"""

from __future__ import annotations

from typing import Any, Optional, Union

import torch


class Device:
    def __init__(self, device_type: str, device_id: int, torch_device: str):
        self.__device_type = device_type
        self.__device_id = device_id
        self.__torch_device = torch_device

    @property
    def device_type(self) -> str:
        return self.__device_type

    @property
    def device_id(self) -> int:
        return self.__device_id

    @property
    def torch_device(self) -> str:
        return self.__torch_device

    def __repr__(self) -> str:
        return f"device({self})"

    def __str__(self) -> str:
        return f"{self.device_type}:{self.device_id}"

    def __eq__(self, other: Any) -> bool:
        if isinstance(other, Device):
            return self.device_type == other.device_type and self.device_id == other.device_id
        if isinstance(other, torch.device):
            return self.device_type == other.type and self.device_id == other.index
        return NotImplemented

    def __hash__(self) -> int:
        return hash((self.device_type, self.device_id))


cpu = Device("cpu", 0, "cpu")
_default_device = cpu
_mapping = {"cpu": cpu}

gpu = None
if torch.cuda.device_count() > 0:
    gpu = Device("gpu", 0, "cuda:0")
    _mapping["gpu"] = gpu
    _mapping["cuda"] = gpu


def get_device() -> Device:
    return _default_device


def sanitize_device(device: Optional[Union[str, Device]] = None) -> Device:
    if device is None:
        return get_device()
    if isinstance(device, Device):
        return device
    try:
        return _mapping[str(device).strip().lower().split(":")[0]]
    except (AttributeError, KeyError, TypeError):
        raise ValueError(f"Unknown device, must be one of {', '.join(_mapping.keys())}")


def use_device(device: Optional[Union[str, Device]] = None) -> None:
    global _default_device
    _default_device = sanitize_device(device)


__all__ = ["Device", "cpu", "get_device", "sanitize_device", "use_device"]
if gpu is not None:
    __all__.append("gpu")
