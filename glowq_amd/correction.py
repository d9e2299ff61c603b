"""Group-shared low-rank correction on top of the W4A16 linear (GlowQ Step 3) and the GlowQ-S
selective variant.

Drop-in for the correction code the reference keeps in its step-3 scripts
(src/step3_eval_dataset.py:409-605; selective patcher src/restoration/step4_evaluate_cumulative.py:99-154):

  `MiniGroupCache`, `AddSVDCorrection(inner, A_q, B_q, role, is_group, group_cache, alpha_svd)`,
  `_role_from_suffix`, `get_parent_module`, `patch_svd_correction_wrappers(model, shared, bmap, alpha_svd)`,
  `patch_svd_correction_wrappers_cumulative(model, shared, bmap, groups_to_patch, alpha_svd)`,
  `_configure_cuda_w4a16_env(args)`.

Naming (kept from the reference): `B_q` is the shared right factor R [rank, K]; `A_q` is the module's
left factor L [N, rank].  The corrected output is  inner(x) + alpha * (x R^T) L^T.

What differs from the reference on purpose is the execution, not the result: the reference runs
inner(x), F.linear(x, B_q), F.linear(r, A_q) and an in-place add per module and shares only r; here
the leader of a group (q / gate) computes r once (`shared_proj`) and runs ONE kernel for all members
of the group with the correction folded into its epilogue.  The members' outputs wait in the group
cache; k / v / up return theirs when called with the same input, and fall back to their own launch
otherwise (the reference's recompute-on-miss, step3_eval_dataset.py:489-498).
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from . import kernels as _kernels
from .linear import KNOBS, CudaW4A16Linear, refresh_env_knobs

_LEADER_USES = {"q": 2, "gate": 1}  # followers that will consume what the leader cached


class MiniGroupCache:
    """One-slot, use-counted cache of the shared projection r (step3_eval_dataset.py:417-444), extended
    with the member outputs of the fused group launch."""

    __slots__ = ("r", "valid", "uses_left", "members", "outputs", "x_key", "x_hold")

    def __init__(self):
        self.r: Optional[torch.Tensor] = None
        self.valid: bool = False
        self.uses_left: int = 0
        self.members: List["AddSVDCorrection"] = []
        self.outputs: Dict[int, torch.Tensor] = {}
        self.x_key = None
        self.x_hold = None  # the leader's input, kept alive so that its address cannot be reused meanwhile

    def set(self, r: torch.Tensor, uses: int):
        self.r = r
        self.valid = True
        self.uses_left = uses

    def consume(self):
        if self.valid and self.uses_left > 0:
            self.uses_left -= 1
            out = self.r
            if self.uses_left == 0:
                self.valid = False
                self.r = None
                self.x_key = None
                self.x_hold = None
            return out, True
        return None, False

    def clear(self):
        self.r = None
        self.valid = False
        self.uses_left = 0
        self.outputs = {}
        self.x_key = None
        self.x_hold = None

    # -- extensions ---------------------------------------------------------------------------------
    def register(self, wrapper: "AddSVDCorrection") -> None:
        if all(w is not wrapper for w in self.members):
            self.members.append(wrapper)

    def take_output(self, wrapper: "AddSVDCorrection"):
        return self.outputs.pop(id(wrapper), None)


def _x_key(x2d: torch.Tensor):
    return (x2d.data_ptr(), tuple(x2d.shape), x2d._version, x2d.device)


class AddSVDCorrection(nn.Module):
    def __init__(self, inner: nn.Module, A_q: torch.Tensor, B_q: torch.Tensor, role: str, is_group: bool,
                 group_cache: Optional[MiniGroupCache], alpha_svd: float = 1.0):
        super().__init__()
        self.inner = inner
        self.register_buffer("A_q", A_q.to(torch.float16).contiguous(), persistent=False)
        self.register_buffer("B_q", B_q.to(torch.float16).contiguous(), persistent=False)
        self.role = role
        self.is_group = is_group
        self.group_cache = group_cache
        self.alpha_svd = alpha_svd
        if is_group and group_cache is not None and hasattr(group_cache, "register"):
            group_cache.register(self)

    # -- checks ---------------------------------------------------------------------------------------
    def _shapes_ok(self) -> bool:
        A, B = self._buffers["A_q"], self._buffers["B_q"]
        memo = self.__dict__.get("_shapes_memo")
        if memo is not None and memo[0] is A and memo[1] is B:  # a tensor's shape does not change under the same object
            return memo[2]
        inner = self.inner
        ok = (A.dim() == 2 and B.dim() == 2 and A.size(1) == B.size(0)
              and A.size(0) == inner.out_features and B.size(1) == inner.in_features)
        self.__dict__["_shapes_memo"] = (A, B, ok)
        return ok

    def _same_right_factor(self, lead: "AddSVDCorrection") -> bool:
        """True when both wrappers hold the same R.  Wrappers built from one artifact tensor share storage;
        after a module-wide .to() each holds its own copy, so contents are compared once and remembered."""
        pa, pb = self.B_q.data_ptr(), lead.B_q.data_ptr()
        if pa == pb:
            return True
        memo = self.__dict__.setdefault("_r_equal_memo", {})
        if (pa, pb) not in memo:
            memo[(pa, pb)] = (self.B_q.shape == lead.B_q.shape and self.B_q.device == lead.B_q.device
                              and bool(torch.equal(self.B_q, lead.B_q)))
        return memo[(pa, pb)]

    def _fusable_with(self, lead: "AddSVDCorrection") -> bool:
        a, b = self.inner, lead.inner
        return (isinstance(a, CudaW4A16Linear) and self.alpha_svd == lead.alpha_svd
                and a.in_features == b.in_features and a.group_size == b.group_size
                and a.qweight_i32.device == b.qweight_i32.device and self._shapes_ok()
                and self._same_right_factor(lead))

    # -- execution ------------------------------------------------------------------------------------
    def _apply(self, fn, *args, **kwargs):
        self.__dict__.pop("_prepared_groups", None)  # descriptors hold the addresses of A_q / B_q
        _kernels.bump_generation()
        return super()._apply(fn, *args, **kwargs)

    def _prepared(self, ext, wrappers, corrected: bool):
        """The launch description of `wrappers` (this one first) with this wrapper's right factor: members validated,
        descriptors and side streams built once and kept until a tensor moves or a factor is replaced."""
        key = (tuple(id(w) for w in wrappers), float(self.alpha_svd), corrected)
        cache = self.__dict__.setdefault("_prepared_groups", {})
        hit = cache.get(key)
        # every tensor whose address sits in the descriptors: a buffer replaced by assignment (re-quantisation,
        # load_state_dict(assign=True), a follower's factor swapped) rebuilds them
        # (read out of the modules' buffer tables: nn.Module's attribute lookup costs several times a dict access)
        ptrs = [self._buffers["B_q"].data_ptr()]
        for w in wrappers:
            inner = w._modules["inner"]
            ib, bias = inner._buffers, inner._parameters.get("bias")
            ptrs += (w._buffers["A_q"].data_ptr(), ib["qweight_i32"].data_ptr(), ib["scales_f16"].data_ptr(), ib["qzeros_i32"].data_ptr(),
                     bias.data_ptr() if bias is not None else 0)
        if hit is not None and hit[0] == ptrs and hit[1].generation == _kernels.generation():
            return hit[1]
        members = []
        for w in wrappers:
            m = w.inner._member(w.A_q if corrected else None)
            m["bias"] = w.inner.bias.data if w.inner.bias is not None else None
            members.append(m)
        pg = _kernels.PreparedGroup(ext, members, self.inner.in_features, self.inner.group_size,
                                    float(self.alpha_svd) if corrected else 0.0, R=self.B_q if corrected else None)
        if len(cache) >= 4:
            cache.clear()
        cache[key] = (ptrs, pg)
        return pg

    def _finish(self, y2d: torch.Tensor, lead_shape) -> torch.Tensor:
        if y2d.dtype != KNOBS.out_dtype:
            y2d = y2d.to(KNOBS.out_dtype)
        return y2d.reshape(*lead_shape, self.inner.out_features)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        inner = self.inner
        KNOBS.sync()
        if self.alpha_svd == 0.0:
            # the reference returns inner(x) untouched (step3_eval_dataset.py:473-474)
            return inner(x)
        if not isinstance(inner, CudaW4A16Linear):
            raise RuntimeError("AddSVDCorrection: the wrapped module must be a CudaW4A16Linear")
        if not self._shapes_ok():
            # the reference swallows the shape error of the correction and returns the uncorrected output
            return inner(x)

        lead_shape = x.shape[:-1]
        x2d = inner._as_rows(x)
        inner._require_gpu(x2d)
        ext = inner._get_ext()
        cache = self.group_cache if self.is_group else None

        if cache is not None and self.role in ("k", "v", "up"):
            key = _x_key(x2d)
            same_x = cache.x_key == key
            r, ok = cache.consume()
            if ok and same_x:
                y = cache.take_output(self)
                if y is not None:
                    return self._finish(y, lead_shape)
            pg = self._prepared(ext, [self], True)
            if ok and same_x and r is not None:
                return self._finish(pg.run(x2d, r=r, project=False)[0], lead_shape)
            return self._finish(pg.run(x2d)[0], lead_shape)  # the reference's recompute-on-miss: r from this module's own R

        if cache is not None and self.role in _LEADER_USES:
            # who joins the leader's launch is decided once per state of the group (members, their alpha switches,
            # tensors not moved since), not on every call
            state = (_kernels.generation(), tuple((id(w), w.alpha_svd) for w in cache.members), self.B_q.data_ptr())
            memo = self.__dict__.get("_group_memo")
            if memo is None or memo[0] != state:
                followers = [w for w in cache.members if w is not self and w._fusable_with(self)]
                memo = (state, [self] + followers[: ext_max_members() - 1])
                self.__dict__["_group_memo"] = memo
            group = memo[1]
            pg = self._prepared(ext, group, True)
            outs = pg.run(x2d)  # r = x R^T and every member of the group in one call
            cache.clear()
            cache.set(pg.last_r, _LEADER_USES[self.role])
            cache.x_key = _x_key(x2d)
            cache.x_hold = x2d
            for w, y in zip(group[1:], outs[1:]):
                cache.outputs[id(w)] = y
            return self._finish(outs[0], lead_shape)
        return self._finish(self._prepared(ext, [self], True).run(x2d)[0], lead_shape)


def ext_max_members() -> int:
    from .kernels import MAX_MEMBERS
    return MAX_MEMBERS


def _role_from_suffix(sfx: str) -> str:
    for tail, role in (("q_proj", "q"), ("k_proj", "k"), ("v_proj", "v"), ("gate_proj", "gate"), ("up_proj", "up")):
        if sfx.endswith(tail):
            return role
    return "solo"


def get_parent_module(model, name: str):
    *path, leaf = name.split(".")
    parent = model
    for p in path:
        parent = getattr(parent, p)
    return parent, leaf


def _plan_entry(weight_name: str, bkey: str, cumulative: bool):
    """(module_name, group key, key of the left factor, role, is_group) for one b_ref_map entry
    (artifact key scheme: src/step2_rsvd.py:487-494,519-522)."""
    module_name = weight_name.replace(".weight", "")
    if "B_shared" in bkey:
        gkey = bkey.replace(".B_shared", "")
        suffix = module_name.split(".")[-1]
        return module_name, gkey, f"{gkey}.{suffix}.A", _role_from_suffix(suffix), True
    gkey = bkey.rsplit(".", 1)[0] if cumulative else bkey.replace(".B", "")
    return module_name, gkey, gkey + ".A", "solo", False


def _patch(model, shared, bmap, alpha_svd, groups_to_patch, verbose: bool):
    caches: Dict[str, MiniGroupCache] = {}
    patched = skipped = 0
    for weight_name, bkey in bmap.items():
        module_name, gkey, a_key, role, is_group = _plan_entry(weight_name, bkey, groups_to_patch is not None)
        if groups_to_patch is not None and gkey not in groups_to_patch:
            continue
        A_q, B_q = shared.get(a_key), shared.get(bkey)
        if A_q is None or B_q is None:
            skipped += 1
            continue
        try:
            parent, leaf = get_parent_module(model, module_name)
            inner = getattr(parent, leaf)
        except AttributeError as e:
            if verbose:
                print(f"AttributeError for {module_name}: {e}")
            skipped += 1
            continue
        if not isinstance(inner, CudaW4A16Linear):
            skipped += 1
            continue
        cache = caches.setdefault(gkey, MiniGroupCache()) if is_group else None
        setattr(parent, leaf, AddSVDCorrection(inner, A_q, B_q, role=role, is_group=is_group, group_cache=cache,
                                               alpha_svd=alpha_svd))
        patched += 1
    if verbose:
        print(f"SVD Correction Patching Summary: {patched} patched, {skipped} skipped")
    return model


def patch_svd_correction_wrappers(model, shared, bmap, alpha_svd=1.0):
    """Wraps every quantised linear named in `bmap` (weight name -> key of its right factor in `shared`)
    with `AddSVDCorrection`; q/k/v and gate/up of a layer share one `MiniGroupCache`
    (step3_eval_dataset.py:535-605)."""
    return _patch(model, shared, bmap, alpha_svd, None, verbose=True)


def patch_svd_correction_wrappers_cumulative(model, shared, bmap, groups_to_patch: set, alpha_svd=1.0):
    """GlowQ-S: only modules whose group key is in `groups_to_patch` get the correction, the others stay
    bare quantised linears (restoration/step4_evaluate_cumulative.py:99-154)."""
    return _patch(model, shared, bmap, alpha_svd, set(groups_to_patch), verbose=False)


def _configure_cuda_w4a16_env(args) -> None:
    """CLI flags -> `W4A16_*` environment knobs, before the model is converted (step3_eval_dataset.py:43-74)."""
    if not getattr(args, "use_cuda_w4a16", False):
        return
    env = os.environ
    env.setdefault("W4A16_KERNEL_OUT_DTYPE", "fp16")
    env.setdefault("W4A16_GEMM_CUDA", "1")
    env.setdefault("W4A16_DEQUANT_CACHE", "0")
    if getattr(args, "cuda_w4a16_kernel_out_dtype", None):
        env["W4A16_KERNEL_OUT_DTYPE"] = args.cuda_w4a16_kernel_out_dtype
    for attr, name in (("cuda_w4a16_gemv_m_max", "W4A16_GEMV_M_MAX"), ("cuda_w4a16_dequant_chunk", "W4A16_DEQUANT_CHUNK")):
        if getattr(args, attr, None) is not None:
            env[name] = str(int(getattr(args, attr)))
    if getattr(args, "cuda_w4a16_dequant_cache", False):
        env["W4A16_DEQUANT_CACHE"] = "1"
    if getattr(args, "cuda_w4a16_force_gemm", False):
        env["W4A16_FORCE_GEMM"] = "1"
        env.pop("W4A16_FORCE_GEMV", None)
    if getattr(args, "cuda_w4a16_force_gemv", False):
        env["W4A16_FORCE_GEMV"] = "1"
        env.pop("W4A16_FORCE_GEMM", None)
    refresh_env_knobs()  # the modules read the switches from a cache, not from the environment on every call
    print("[CUDA W4A16] env:"
          f" out_dtype={env.get('W4A16_KERNEL_OUT_DTYPE')}"
          f", gemv_m_max={env.get('W4A16_GEMV_M_MAX', '(default)')}"
          f", force_gemm={env.get('W4A16_FORCE_GEMM', '0')}"
          f", force_gemv={env.get('W4A16_FORCE_GEMV', '0')}"
          f", dequant_chunk={env.get('W4A16_DEQUANT_CHUNK', '(default)')}"
          f", dequant_cache={env.get('W4A16_DEQUANT_CACHE', '0')}")


__all__ = ["MiniGroupCache", "AddSVDCorrection", "patch_svd_correction_wrappers",
           "patch_svd_correction_wrappers_cumulative", "get_parent_module", "_role_from_suffix",
           "_configure_cuda_w4a16_env"]
