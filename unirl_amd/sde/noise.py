"""Initial-noise (x_T) recipe with the call contract of ``unirl/sde/noise.py``.

``_derive_group_seed`` (:26-29), ``generate_shared_noise`` (:32-97), ``generate_latents``
(:100-152) and ``regen_initial_noise`` (:155-187) keep their signatures, errors and -- the point of
the recipe -- their bytes: ``regen_initial_noise`` draws every noise group on the CPU in fp32 from
a ``torch.Generator`` seeded with ``blake2b(f"{base_seed}::{group_id}")``, so all engines start a
rollout from the same x_T.  The draw itself therefore stays on the host.  What changes is what
happens after it: the reference stacks one copy of the draw per SAMPLE on the host and uploads
and casts the whole ``[B, ...]`` batch; here only the ``U`` unique draws cross PCIe, from a pinned
staging buffer, and one kernel (``unirl_expand_groups``) replicates them to the ``B`` samples and
applies the final dtype cast.  With 16 samples per prompt that is 16x less host-to-device traffic
and no ``[B, ...]`` host tensor.
"""

from __future__ import annotations

import hashlib
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops

# Inclusive maximum accepted by torch.Generator.manual_seed.
MAX_TORCH_SEED = (1 << 63) - 1


def _derive_group_seed(base_seed: int, group_id: str) -> int:
    payload = f"{int(base_seed)}::{str(group_id)}".encode("utf-8")
    digest = hashlib.blake2b(payload, digest_size=8).digest()
    return int.from_bytes(digest, byteorder="big", signed=False) % (MAX_TORCH_SEED + 1)


class _PinnedStaging:
    """One growing pinned host buffer per device; a copy out of it must finish before it is refilled."""

    def __init__(self) -> None:
        self.buf: Optional[torch.Tensor] = None
        self.busy: Optional[torch.cuda.Event] = None

    def take(self, numel: int) -> torch.Tensor:
        if self.busy is not None:
            self.busy.synchronize()
            self.busy = None
        if self.buf is None or self.buf.numel() < numel:
            self.buf = torch.empty(numel, dtype=torch.float32, pin_memory=True)
        return self.buf[:numel]

    def sent(self, device: torch.device) -> None:
        self.busy = torch.cuda.Event()
        self.busy.record(torch.cuda.current_stream(device))


_staging: Dict[int, _PinnedStaging] = {}


def _unique_groups(noise_group_ids: List) -> Tuple[List[str], List[int]]:
    """Distinct group ids in first-appearance order, and each sample's index into them."""
    slot: Dict[str, int] = {}
    group_of: List[int] = []
    for raw in noise_group_ids:
        gid = str(raw)
        if gid not in slot:
            slot[gid] = len(slot)
        group_of.append(slot[gid])
    return list(slot), group_of


def generate_shared_noise(
    batch_size: int,
    latent_shape: Tuple[int, ...],
    device: torch.device,
    dtype: torch.dtype = torch.float32,
    noise_group_ids: Optional[List[str]] = None,
    base_seed: Optional[int] = None,
) -> torch.Tensor:
    """``[batch_size, *latent_shape]`` noise in which samples of one ``noise_group_id`` share a draw.

    Like the reference, each group is drawn on ``device`` in ``dtype`` -- from a generator seeded
    with ``_derive_group_seed(base_seed, group_id)`` when ``base_seed`` is given -- in order of
    first appearance.  On a HIP device the groups are replicated to the samples by one kernel
    (fp32 / bf16 / fp16); other dtypes and CPU tensors are stacked as the reference does.
    """
    if not isinstance(noise_group_ids, list) or len(noise_group_ids) != batch_size:
        raise ValueError(
            "generate_shared_noise requires explicit noise_group_ids aligned to batch_size. "
            f"Got batch_size={batch_size}, noise_group_ids_len="
            f"{len(noise_group_ids) if isinstance(noise_group_ids, list) else None}."
        )
    device = torch.device(device)
    groups, group_of = _unique_groups(noise_group_ids)
    draws: List[torch.Tensor] = []
    for gid in groups:
        if base_seed is None:
            draws.append(torch.randn(*latent_shape, device=device, dtype=dtype))
        else:
            gen = torch.Generator(device=device)
            gen.manual_seed(_derive_group_seed(base_seed, gid))
            draws.append(torch.randn(*latent_shape, device=device, dtype=dtype, generator=gen))
    if device.type == "cuda" and dtype == torch.float32 and draws:
        unique = torch.stack(draws, dim=0)
        return ops.expand_groups(unique, torch.tensor(group_of, dtype=torch.int64, device=device), dtype)
    if not draws:
        return torch.empty((0,) + tuple(latent_shape), device=device, dtype=dtype)
    return torch.stack([draws[k] for k in group_of], dim=0)


def generate_latents(
    batch_size: int,
    latent_shape: Tuple[int, ...],
    device: torch.device,
    dtype: torch.dtype = torch.float32,
    init_same_noise: bool = False,
    samples_per_prompt: int = 1,
    noise_group_ids: Optional[List[str]] = None,
    base_seed: Optional[int] = None,
) -> torch.Tensor:
    """Initial latents: shared per group when ``init_same_noise``, plain ``randn`` otherwise."""
    del samples_per_prompt  # geometry hint kept for API compatibility
    if init_same_noise:
        assert base_seed is not None and noise_group_ids is not None, (
            "generate_latents requires both base_seed and noise_group_ids when init_same_noise=True."
        )
        return generate_shared_noise(
            batch_size=batch_size, latent_shape=latent_shape, device=device, dtype=dtype,
            noise_group_ids=noise_group_ids, base_seed=base_seed,
        )
    return torch.randn(batch_size, *latent_shape, device=device, dtype=dtype)


def regen_initial_noise(
    noise_group_ids: List[str],
    base_seed: int,
    latent_shape: Tuple[int, ...],
    device: torch.device,
    dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """x_T from the driver's recipe, byte-identical on every engine: each group is drawn on the
    CPU in fp32 from its derived seed; moving to ``device`` and casting to ``dtype`` come last."""
    device = torch.device(device)
    gids = list(noise_group_ids)
    shape = tuple(int(s) for s in latent_shape)
    if device.type != "cuda" or dtype not in (torch.float32, torch.bfloat16, torch.float16):
        x = generate_shared_noise(len(gids), shape, torch.device("cpu"), torch.float32, gids, int(base_seed))
        return x.to(device=device, dtype=dtype)
    groups, group_of = _unique_groups(gids)
    per = 1
    for s in shape:
        per *= s
    if not groups or per == 0:
        return torch.empty((len(gids),) + shape, device=device, dtype=dtype)
    index = device.index if device.index is not None else torch.cuda.current_device()
    device = torch.device("cuda", index)
    stage = _staging.setdefault(index, _PinnedStaging())
    host = stage.take(len(groups) * per).view((len(groups),) + shape)
    for u, gid in enumerate(groups):
        gen = torch.Generator(device="cpu")
        gen.manual_seed(_derive_group_seed(int(base_seed), gid))
        host[u].copy_(torch.randn(*shape, device="cpu", dtype=torch.float32, generator=gen))
    unique = host.to(device, non_blocking=True)
    stage.sent(device)
    return ops.expand_groups(unique, torch.tensor(group_of, dtype=torch.int64).to(device), dtype)


__all__ = [
    "MAX_TORCH_SEED",
    "generate_latents",
    "generate_shared_noise",
    "regen_initial_noise",
]
