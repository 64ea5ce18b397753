"""Position encodings. They act on the packed query/key/value rows of a step and
hand keys and values to the cache in the same pass."""
import torch

from .. import memory

from ..registry import register_part
from ..status import EINVAL, fail
from .base import Part


@register_part("position", "rotary")
class Rotary(Part):
    """Rotation of pairs ``(i, i + rot_dim/2)`` of each head by the angle
    ``pos * theta^(-2i/rot_dim)`` (split-half pairing, src/model.c:468-493; the
    reference builds the angle by a running fp32 product, here it is one fp32
    product of the position and a table rounded from fp64). Dimensions from
    ``rot_dim`` on pass through. Values are not rotated; keys are stored rotated
    (src/model.c:596-600)."""
    graph_safe = True


    def __init__(self, head_dim, rot_dim, theta, pairing="split_half", prefix=""):
        super().__init__(prefix)
        if pairing != "split_half":
            fail(EINVAL, f"rotary pairing '{pairing}' is not implemented")
        if rot_dim % 2 or not 0 < rot_dim <= head_dim:
            fail(EINVAL, f"rotary rot_dim {rot_dim} must be even and within head_dim {head_dim}")
        self.head_dim = head_dim
        self.rot_dim = rot_dim
        self.theta = float(theta)
        self.inv_freq = None

    def bind(self, params, ops):
        def table():
            i = torch.arange(self.rot_dim // 2, dtype=torch.float64)
            inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / self.rot_dim)
            return memory.to_device(inv.to(torch.float32), ops.device, "rotary frequencies")
        # layers with the same rotation share one table (and with it what a step derives from it once for all of them)
        self.inv_freq = ops.shared(("rotary frequencies", self.rot_dim, self.theta), table)

    def store(self, ops, step, qkv, n_heads, n_kv_heads, cache, write, v_head_dim=None):
        """Rotates the queries (and keys) inside ``qkv`` at each token's position;
        if ``write``, puts each token's rotated key and its value into its cache row.
        ``v_head_dim``: the size of a value head where it is not the keys'."""
        ops.rope_store(qkv, step.positions, self.inv_freq, self.rot_dim, n_heads, n_kv_heads,
                       self.head_dim, cache, step.group(cache.group).slot_map if write else None, v_head_dim=v_head_dim)


@register_part("position", "none")
class NoPosition(Part):
    """No position encoding: keys and values go to the cache as they are."""
    graph_safe = True


    def __init__(self, head_dim, prefix=""):
        super().__init__(prefix)
        self.head_dim = head_dim

    def store(self, ops, step, qkv, n_heads, n_kv_heads, cache, write, v_head_dim=None):
        if write:
            ops.rope_store(qkv, step.positions, None, 0, n_heads, n_kv_heads, self.head_dim,
                           cache, step.group(cache.group).slot_map, v_head_dim=v_head_dim)
