"""Configuration types of the Mamba-1 path, mirroring the reference's names.

MambaConfig / ScanMode follow src/config.rs:6-186, WeightDtype follows
src/mamba_ssm/gpu/dtype.rs:12-44 (same variant order, used as the C ABI code).
"""
from __future__ import annotations

import enum
from dataclasses import dataclass

from . import _lib


class WeightDtype(enum.IntEnum):
    F32 = 0
    F16 = 1
    BF16 = 2

    def size_bytes(self) -> int:
        return 4 if self is WeightDtype.F32 else 2

    def torch_dtype(self):
        import torch
        return {WeightDtype.F32: torch.float32, WeightDtype.F16: torch.float16, WeightDtype.BF16: torch.bfloat16}[self]

    @staticmethod
    def from_torch(dt) -> "WeightDtype":
        import torch
        try:
            return {torch.float32: WeightDtype.F32, torch.float16: WeightDtype.F16, torch.bfloat16: WeightDtype.BF16}[dt]
        except KeyError:
            raise ValueError(f"unsupported activation dtype {dt}") from None


class ScanMode(enum.IntEnum):
    SEQUENTIAL = 0
    PARALLEL = 1
    AUTO = 2

    def use_parallel(self, seq_len: int, d_state: int) -> bool:
        """ScanMode::use_parallel (src/config.rs:28-37), answered by the library."""
        return bool(_lib.load().mrs_scan_use_parallel(int(self), seq_len, d_state))

    def resolve(self, seq_len: int, d_state: int) -> "ScanMode":
        return ScanMode.PARALLEL if self.use_parallel(seq_len, d_state) else ScanMode.SEQUENTIAL


# Auto threshold: sequential at or below, parallel above (src/config.rs:21).
PARALLEL_SCAN_THRESHOLD = 256


@dataclass(frozen=True)
class MambaConfig:
    d_model: int = 128
    d_state: int = 16
    d_conv: int = 4
    expand: int = 2
    n_layers: int = 3
    scan_mode: ScanMode = ScanMode.AUTO
    rms_norm_eps: float = 1e-5

    def d_inner(self) -> int:
        return self.expand * self.d_model

    def dt_rank(self) -> int:
        return -(-self.d_model // 16)

    def xdbl_dim(self) -> int:
        return self.dt_rank() + 2 * self.d_state

    def validate(self) -> None:
        """Same bounds and messages as MambaConfig::validate (src/config.rs:108-170); raises ValueError."""
        for name in ("d_model", "d_state", "d_conv", "expand", "n_layers"):
            if getattr(self, name) == 0:
                raise ValueError(f"{name} must be > 0")
        if self.d_model > (1 << 20):
            raise ValueError(f"d_model ({self.d_model}) must be <= 2^20")
        if self.n_layers > 4096:
            raise ValueError(f"n_layers ({self.n_layers}) must be <= 4096")
        if self.d_inner() > 65535:
            raise ValueError(f"d_inner ({self.d_inner()}) must be <= 65535")
        if self.d_state > 256:
            raise ValueError(f"d_state ({self.d_state}) must be <= 256")
        if self.d_conv > 8:
            raise ValueError(f"d_conv ({self.d_conv}) must be <= 8")
        if self.d_inner() % 4 != 0:
            raise ValueError(f"d_inner ({self.d_inner()}) must be divisible by 4")
