"""One launch for sibling linears that read the same activation (q/k/v, gate/up, qkv/z): the machinery both pack formats
share.  A format supplies `combine(members) -> (fused linear, row split points)`; the members of a group are replaced by
thin modules that hand out their slice of the fused result.

Which siblings are fed the same tensor is a property of the model families the reference serves
(src/qv_band/formats/qvb8r/fuse.py:17-21)."""
from __future__ import annotations

import torch
import torch.nn as nn

# (attribute of a layer that owns the siblings, names of the siblings)
SAME_INPUT_GROUPS = (
    ("self_attn", ("q_proj", "k_proj", "v_proj")),
    ("linear_attn", ("in_proj_qkv", "in_proj_z")),
    ("mlp", ("gate_proj", "up_proj")),
)


class FusedGroup(nn.Module):
    """Holds the fused linear of one group.  The first member that is called with a tensor computes every member's
    output; the others take theirs from that result."""

    def __init__(self, lin: nn.Module, splits: list[int]):
        super().__init__()
        self.lin, self.splits = lin, list(splits)
        self._x = None
        self._ver = None
        self._outs = None
        self._left: set = set()

    def forward(self, x):
        """All members' outputs for `x`, as views of one result."""
        return torch.tensor_split(self.lin(x), self.splits, -1)

    def get(self, x, i):
        # A stored result is handed out only for the SAME tensor object (kept alive here, so its storage cannot be reused
        # by another tensor meanwhile), unmodified since (its version counter), and only until every member has taken
        # its part once (fuse.py:64-77 of the reference).  This reuse lives in Python: under graph replay capture
        # forward() instead.
        if self._x is not x or x._version != self._ver or i not in self._left:
            self._outs = self.forward(x)
            self._x, self._ver = x, x._version
            self._left = set(range(len(self._outs)))
        self._left.discard(i)
        out = self._outs[i]
        if not self._left:
            self._x = self._outs = None
        return out


class FusedMember(nn.Module):
    """Stands where a member linear stood: same in/out features, forwards to the group.  `bias`: None when the fused linear
    adds the members' biases itself, else this member's own, added here."""

    def __init__(self, group: FusedGroup, i: int, in_features: int, out_features: int, bias=None):
        super().__init__()
        object.__setattr__(self, "group", group)       # shared by the members: kept out of the module tree
        self.i, self.in_features, self.out_features = i, in_features, out_features
        self.bias = bias

    def forward(self, x):
        y = self.group.get(x, self.i)
        return y if self.bias is None else y + self.bias.to(y.dtype)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, fused member {self.i}"


def fuse_groups(model: nn.Module, eligible, combine, attr: str, member_bias=lambda m: None) -> int:
    """Replaces every same-input group whose members all satisfy `eligible(owner, names)` by FusedMembers of one
    FusedGroup built by `combine(list of members)`.  The group is registered once, as `attr` of the layer that owns the
    siblings.  Returns the number of groups fused.

    No list of the model's modules is kept while groups are replaced, and a group's separate members are released before
    the next group is built: otherwise the separate and the fused copies of the whole model would exist side by side."""
    owners = [(owner, names) for parent in model.modules() for sub, names in SAME_INPUT_GROUPS
              if (owner := getattr(parent, sub, None)) is not None and eligible(owner, names)]
    done = 0
    for owner, names in owners:
        members = [getattr(owner, a) for a in names]
        shapes = [(m.in_features, m.out_features, member_bias(m)) for m in members]
        for a in names:
            setattr(owner, a, None)
        lin, splits = combine(members)
        del members
        group = FusedGroup(lin, splits)
        setattr(owner, attr, group)
        for i, (a, (pin, pout, b)) in enumerate(zip(names, shapes)):
            setattr(owner, a, FusedMember(group, i, pin, pout, b))
        done += 1
    if done and torch.cuda.is_available():
        torch.cuda.empty_cache()
    return done
