"""The card kernels' typed launchers for this path: the surface of the reference's generated btb/engine/card_launch.py
(`Launcher` :428-440, `ptr` :443-446, one function a kernel, `CardLaunch` :2720-2736) restricted to the kernels this
library serves. A function takes a launcher, then - for a kernel family instantiated per head width or per row count -
the variant (`D`, `M`), then the CUDA launch geometry (`grid`, `block`), then the kernel's parameters in the order of
its `extern "C"` declaration (native/cuda/btb_kernels.cu, btb_gemv_mma.cuh, btb_attn_flash.cuh), each typed by its role;
it packs them as ctypes values and hands them to `launcher.launch(name, grid, block, args, stream, shared)`.
`CardLaunch` carries every function as a method, so `k.btb_attn_flash(D, ...)` is `btb_attn_flash(k, D, ...)` and the
reference's `_card_body` (btb/engine/cuda.py:1601-1837) can be handed any object that mixes `CardLaunch` in and
implements `launch` - `btb_amd.native.HipCard` does.

Where the reference writes the functions out one by one (its build generates them from the CUDA sources), here one
table states every kernel's parameters and the functions are made from it.
"""

from __future__ import annotations

import ctypes
from collections.abc import Callable, Sequence
from typing import Any, NewType, Protocol, TypeVar

Dim3 = tuple[int, int, int]
_R = TypeVar("_R")

_PACK = {"p": ctypes.c_void_p, "i": ctypes.c_int, "f": ctypes.c_float, "l": ctypes.c_longlong}

# kernel family -> (variant, parameters). variant "": one kernel of that name; "D": `<name>_d{D}` for a head width;
# "M": `<name>_m{M}` for a row count. A parameter is name:Role:kind, kind p a card address, i an int, f a float, l a
# 64-bit int - the reference kernel's own list, in its order.
SPEC: dict[str, tuple[str, str]] = {
    "btb_add_rmsnorm": ("", "h:Residual:p y:BlockOut:p w:NormWeight:p eps:NormEps:f x:Normed:p H:Hidden:i "
                            "centered:NormCentered:i"),
    "btb_attn_flash": ("D", "q:Query:p K:KCache:p V:VCache:p out:AttnOut:p n0p:PrefixLen:p par:TreeParents:p T:Rows:i "
                            "Hq:QHeads:i Hk:KvHeads:i hs:CacheHeadStride:i rs:CacheRowStride:i scale:AttnScale:f "
                            "part_m:PartMax:p part_l:PartSum:p part_acc:PartAcc:p cnt:Arrivals:p win:Window:i tbl:RowMap:p"),
    "btb_attn_flash_rows": ("D", "q:Query:p K:KCache:p V:VCache:p out:AttnOut:p rw:RowsLayout:p T:Rows:i Hq:QHeads:i "
                                 "Hk:KvHeads:i hs:CacheHeadStride:i rs:CacheRowStride:i scale:AttnScale:f part_m:PartMax:p "
                                 "part_l:PartSum:p part_acc:PartAcc:p cnt:Arrivals:p win:Window:i"),
    "btb_gemv_bf16": ("M", "w:Weight:p x:MatIn:p y:MatOut:p R:OutDim:i C:InDim:i"),
    "btb_gemv_silu_bf16": ("M", "w:Weight:p gu:GateUp:p y:MatOut:p R:OutDim:i C:InDim:i"),
    "btb_gemv_lane16_f32": ("M", "w:Weight:p x:MatInF32:p y:MatOutF32:p R:OutDim:i C:InDim:i"),
    "btb_gemv_lane16_mx4_f32": ("M", "blocks:Mx4Blocks:p scales:Mx4Scales:p x:MatInF32:p y:MatOutF32:p R:OutDim:i "
                                     "C:InDim:i"),
    "btb_gemv_mma_bf16": ("", "w:Weight:p x:MatIn:p y:MatOut:p R:OutDim:i C:InDim:i M:Rows:i"),
    "btb_gemv_mma8_bf16": ("", "w:Weight:p x:MatIn:p y:MatOut:p R:OutDim:i C:InDim:i M:Rows:i"),
    "btb_gemv_mma_glu_silu": ("", "w:Weight:p x:MatIn:p m:MlpAct:p I:Intermediate:i C:InDim:i M:Rows:i"),
    "btb_moe_route": ("", "logits:RouterLogits:p ls:RouterStride:i E:Experts:i k:TopExperts:i idx:ExpertIds:p "
                          "w:ExpertWeights:p hidx:HostExpertIds:p hw:HostExpertWeights:p cnt:RouteCount:p seq:RouteSeq:p "
                          "hseq:HostRouteSeq:p"),
    "btb_mx4_widen": ("", "blocks:Mx4Blocks:p scales:Mx4Scales:p seats:Seats:p groups:Mx4Groups:l out:Widened:p"),
    "btb_norm_rope_kv": ("D", "qkv:Qkv:p wq:QNorm:p wk:KNorm:p eps:NormEps:f cos_t:RopeCos:p sin_t:RopeSin:p "
                              "n0p:PrefixLen:p depth:Depths:p K:KCache:p V:VCache:p qo:Query:p T:Rows:i Hq:QHeads:i "
                              "Hk:KvHeads:i hs:CacheHeadStride:i rs:CacheRowStride:i centered:NormCentered:i"),
    "btb_norm_rope_kv_rows": ("D", "qkv:Qkv:p wq:QNorm:p wk:KNorm:p eps:NormEps:f cos_t:RopeCos:p sin_t:RopeSin:p "
                                   "rw:RowsLayout:p K:KCache:p V:VCache:p qo:Query:p T:Rows:i Hq:QHeads:i Hk:KvHeads:i "
                                   "hs:CacheHeadStride:i rs:CacheRowStride:i centered:NormCentered:i"),
    "btb_norm_rope_kv_tbl": ("D", "qkv:Qkv:p wq:QNorm:p wk:KNorm:p eps:NormEps:f cos_t:RopeCos:p sin_t:RopeSin:p "
                                  "n0p:PrefixLen:p depth:Depths:p K:KCache:p V:VCache:p qo:Query:p T:Rows:i Hq:QHeads:i "
                                  "Hk:KvHeads:i hs:CacheHeadStride:i rs:CacheRowStride:i centered:NormCentered:i "
                                  "tbl:RowMap:p"),
    "btb_publish": ("", "n0:PrefixLen:p ids:StepToken:p out_tok:HostToken:p out_n0:HostLen:p out_ts:HostClock:p"),
    "btb_silu_mul": ("", "gu:GateUp:p m:MlpAct:p T:Rows:i I:Intermediate:i"),
}

VARIANTS = {"D": (64, 128, 256), "M": (1, 2, 4, 8, 16, 32)}


def _parse(params: str) -> list[tuple[str, str, str]]:
    return [tuple(p.split(":")) for p in params.split()]  # type: ignore[misc]


def kernel_names(family: str) -> tuple[str, ...]:
    """the kernels a family stands for: itself, or one a head width / row count"""
    variant, _ = SPEC[family]
    if not variant:
        return (family,)
    return tuple(f"{family}_{variant.lower()}{v}" for v in VARIANTS[variant])


# every kernel name this path serves, a family's at each of its instantiations (the reference's `KERNELS`, :207-425,
# less the kernels of other paths; the attention is built for head_dim 128 only)
KERNELS: tuple[str, ...] = tuple(n for fam in SPEC for n in kernel_names(fam)
                                 if not (fam.startswith("btb_attn_flash") and not n.endswith("_d128")))

# the roles: what a parameter is, as a type of its own over int (the reference's btb/kinds.py, from
# native/cuda/btb_roles.cuh) - `ptr(Query, q)` is q's card address typed as the attention's query rows
ROLES: dict[str, Any] = {}
for _fam, (_v, _params) in SPEC.items():
    for _name, _role, _kind in _parse(_params):
        if _role not in ROLES:
            ROLES[_role] = NewType(_role, float if _kind == "f" else int)
globals().update(ROLES)


class Launcher(Protocol):
    """what launches a kernel: its name, the grid and block, one ctypes value a parameter, the stream, and the bytes of
    dynamic shared memory (btb/engine/card_launch.py:428-440)"""

    def launch(self, name: str, grid: Dim3, block: Dim3, args: Sequence[Any], stream: Any = None,
               shared: int = 0) -> None: ...


def ptr(role: Callable[[int], _R], t: Any) -> _R:
    """tensor `t`'s card address as an argument of `role`; None the null pointer. The address keeps nothing alive"""
    return role(0 if t is None else t.data_ptr())


def _typed(family: str) -> Callable[..., None]:
    variant, params = SPEC[family]
    fields = _parse(params)
    packers = [_PACK[kind] for _, _, kind in fields]
    names = [n for n, _, _ in fields]
    lead = 1 if variant else 0
    order = ([variant] if variant else []) + ["grid", "block"] + names

    def fn(launcher: Launcher, *a: Any, stream: Any = None, shared: int = 0, **kw: Any) -> None:
        want = lead + 2 + len(fields)
        if kw:  # parameters by name, as the reference's functions take them too
            rest = order[len(a):]
            extra = sorted(n for n in kw if n not in rest)
            if extra:
                raise TypeError(f"{family}() got unexpected or repeated arguments {extra}")
            missing = [n for n in rest if n not in kw]
            if missing:
                raise TypeError(f"{family}() is missing {missing}")
            a = a + tuple(kw[n] for n in rest)
        if len(a) != want:
            raise TypeError(f"{family}() takes {want} arguments after the launcher "
                            f"({'the variant ' + variant + ', ' if variant else ''}grid, block, {', '.join(names)}), got {len(a)}")
        if variant:
            v = int(a[0])
            if v not in VARIANTS[variant]:
                raise ValueError(f"{family}: {variant} is one of {VARIANTS[variant]}, got {v}")
            name = f"{family}_{variant.lower()}{v}"
        else:
            name = family
        grid, block = a[lead], a[lead + 1]
        packed = [pack(None if (pack is ctypes.c_void_p and not val) else val)
                  for pack, val in zip(packers, a[lead + 2:])]
        launcher.launch(name, grid, block, packed, stream, shared)

    fn.__name__ = fn.__qualname__ = family
    fn.__doc__ = (f"{family}{'_' + variant.lower() + '{' + variant + '}' if variant else ''}"
                  f"({', '.join(n + ': ' + r for n, r, _ in fields)})")
    return fn


class CardLaunch:
    """the launchers as methods of a card's kernel module, each the function of its name with the module as its
    launcher (btb/engine/card_launch.py:2720-2736); `launch` is the module's to implement"""

    def launch(self, name: str, grid: Dim3, block: Dim3, args: Sequence[Any], stream: Any = None,
               shared: int = 0) -> None:
        raise NotImplementedError

    ptr = staticmethod(ptr)


for _fam in SPEC:
    _f = _typed(_fam)
    globals()[_fam] = _f
    setattr(CardLaunch, _fam, _f)
del _fam, _f, _v, _params, _name, _role, _kind
