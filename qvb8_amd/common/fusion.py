"""One launch for sibling linears that read the same activation (q/k/v, gate/up, qkv/z): the machinery both pack formats
share.  A format supplies `combine(members) -> (fused linear, row split points)`; the members of a group are replaced by
thin modules that hand out their slice of the fused result.

Which siblings are fed the same tensor is a property of the model families the reference serves
(src/qv_band/formats/qvb8r/fuse.py:17-21); what the fused launch must do for its callers -- one product per distinct
input, every member's slice handed out once -- is that of fuse.py:52-119 there.
"""
from __future__ import annotations

import weakref

import torch
import torch.nn as nn

# (attribute of a layer that owns the siblings, names of the siblings)
SAME_INPUT_GROUPS = (
    ("self_attn", ("q_proj", "k_proj", "v_proj")),
    ("linear_attn", ("in_proj_qkv", "in_proj_z")),
    ("mlp", ("gate_proj", "up_proj")),
)


class _Held:
    """The fused result of one input, kept until each member has fetched its part: which tensor it was computed from (a weak
    reference plus the tensor's version counter, so neither a new tensor at the old address nor the old tensor modified in
    place can be mistaken for it), the parts, and one bit per member that has not fetched yet."""
    __slots__ = ("source", "version", "parts", "waiting")

    def __init__(self, x: torch.Tensor, parts):
        self.source, self.version = weakref.ref(x), x._version
        self.parts = parts
        self.waiting = (1 << len(parts)) - 1

    def serves(self, x: torch.Tensor, member: int) -> bool:
        return self.source() is x and x._version == self.version and bool(self.waiting >> member & 1)


class FusedGroup(nn.Module):
    """Holds the fused linear of one group.  The first member called with a tensor makes the one launch for all; the others
    take their slices of that result.  This sharing lives in Python: a graph capture records forward() instead."""

    def __init__(self, lin: nn.Module, splits: list[int]):
        super().__init__()
        self.lin, self.splits = lin, list(splits)
        self._held: _Held | None = None

    def forward(self, x):
        """All members' outputs for `x`, as views of one result."""
        return torch.tensor_split(self.lin(x), self.splits, -1)

    def holding(self) -> bool:
        """Whether a result is still kept for members that have not fetched their part."""
        return self._held is not None

    def part(self, x, member: int):
        held = self._held
        if held is None or not held.serves(x, member):
            held = self._held = _Held(x, self.forward(x))
        held.waiting &= ~(1 << member)
        if held.waiting == 0:                              # every member has its part: nothing is kept alive
            self._held = None
        return held.parts[member]


class FusedMember(nn.Module):
    """Stands where a member linear stood: same in/out features, forwards to the group.  `bias`: None when the fused linear
    adds the members' biases itself, else this member's own, added here."""

    def __init__(self, group: FusedGroup, i: int, in_features: int, out_features: int, bias=None):
        super().__init__()
        self._group = (group,)                             # inside a tuple: the members share it, only its owner registers it
        self.i, self.in_features, self.out_features = i, in_features, out_features
        self.bias = bias

    @property
    def group(self) -> FusedGroup:
        return self._group[0]

    def forward(self, x):
        out = self._group[0].part(x, self.i)
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out

    def extra_repr(self):
        return f"member {self.i} of a fused launch: {self.in_features} -> {self.out_features}"


def _sibling_groups(model: nn.Module, eligible):
    """(owner, names) of every same-input group under `model` whose members all pass `eligible`."""
    found = []
    for parent in model.modules():
        for holder, names in SAME_INPUT_GROUPS:
            owner = getattr(parent, holder, None)
            if owner is not None and eligible(owner, names):
                found.append((owner, names))
    return found


def fuse_groups(model: nn.Module, eligible, combine, attr: str, member_bias=lambda m: None) -> int:
    """Replaces every same-input group whose members all satisfy `eligible(owner, names)` by FusedMembers of one
    FusedGroup built by `combine(list of members)`.  The group is registered once, as `attr` of the layer that owns the
    siblings.  Returns the number of groups fused.

    Only (owner, names) pairs are kept while groups are replaced, and a group's separate members are taken off their owner
    before its fused linear is built: otherwise the separate and the fused copies of the whole model would exist side by
    side."""
    groups = _sibling_groups(model, eligible)
    for owner, names in groups:
        members = []
        for name in names:
            members.append(getattr(owner, name))
            setattr(owner, name, None)
        facts = [(m.in_features, m.out_features, member_bias(m)) for m in members]
        lin, splits = combine(members)
        members.clear()
        group = FusedGroup(lin, splits)
        setattr(owner, attr, group)
        for index, (name, (n_in, n_out, bias)) in enumerate(zip(names, facts)):
            setattr(owner, name, FusedMember(group, index, n_in, n_out, bias))
    if groups and torch.cuda.is_available():
        torch.cuda.empty_cache()
    return len(groups)
