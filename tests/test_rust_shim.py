"""The Rust shim (rust/) cannot be compiled in this image; what can be checked without a toolchain:
every method of the reference's `trait Backend` is implemented in hip.rs, and every sys::cg_* function
it calls is declared in the FFI crate with the argument count the C header declares."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRAIT = "/root/reference/catgrad/src/interpreter/backend/mod.rs"
HIP_RS = os.path.join(ROOT, "rust", "catgrad", "src", "interpreter", "backend", "hip.rs")
SYS_RS = os.path.join(ROOT, "rust", "catgrad-hip-sys", "src", "lib.rs")
HEADER = os.path.join(ROOT, "include", "catgrad_hip.h")

# the 27 methods of trait Backend (catgrad/src/interpreter/backend/mod.rs:26-81) + BackendTensorOps::shape (:84-86)
TRAIT_METHODS = ["zeros", "ndarray_from_vec_f32", "ndarray_from_vec_u32", "cast", "matmul", "add", "sub", "mul",
                 "div", "pow", "lt", "eq", "sin", "cos", "neg", "broadcast", "reshape", "transpose", "max", "sum",
                 "argmax", "topk", "compare", "concat", "index", "slice", "arange", "to_vec"]


def _impl_block(src):
    return src[src.index("\nimpl Backend for HipBackend {"):src.index("#[cfg(test)]")]


def _c_args(header, name):
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)            # declarations only
    m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % re.escape(name), header, re.S)
    assert m, f"{name} not declared in the header"
    args = m.group(1).strip()
    return 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])


def _rust_args(sys_src, name):
    m = re.search(r"pub fn %s\s*\(([^;]*?)\)\s*(->[^;]*)?;" % re.escape(name), sys_src, re.S)
    assert m, f"{name} not declared in catgrad-hip-sys"
    args = m.group(1).strip()
    return 0 if not args else len([a for a in args.split(",") if a.strip()])


def test_method_list_is_the_reference_trait():
    if not os.path.exists(TRAIT):
        pytest.skip("the reference tree is not on this machine")
    src = open(TRAIT).read()
    body = src[src.index("pub trait Backend"):src.index("pub trait BackendTensorOps")]
    assert re.findall(r"^\s*fn (\w+)", body, re.M) == TRAIT_METHODS


def test_every_trait_method_is_implemented_over_the_c_abi():
    impl = _impl_block(open(HIP_RS).read())
    implemented = re.findall(r"^\s*fn (\w+)", impl, re.M)
    assert implemented == TRAIT_METHODS
    for name in TRAIT_METHODS:
        body = impl[impl.index(f"fn {name}("):]
        nxt = re.search(r"\n    fn |\n    /// ", body[1:])
        body = body[:nxt.start() + 1] if nxt else body
        c_name = {"ndarray_from_vec_f32": "cg_from_f32", "ndarray_from_vec_u32": "cg_from_u32",
                  "to_vec": "cg_to_f32"}.get(name, "cg_" + name)
        assert f"sys::{c_name}" in body, f"{name} does not forward to {c_name}"
    assert "impl BackendTensorOps for HipTensor" in open(HIP_RS).read()
    assert "impl fmt::Debug for HipBackend" in open(HIP_RS).read()          # Backend: Clone + Debug


def test_ffi_declarations_match_the_header():
    header, sys_src, hip = open(HEADER).read(), open(SYS_RS).read(), open(HIP_RS).read()
    used = set(re.findall(r"sys::(cg_[a-z0-9_]+)\s*[(,)]", hip))
    used -= {"cg_out", "cg_backend", "cg_tensor"}                       # the opaque types
    assert len(used) >= 35
    for name in sorted(used):
        assert _rust_args(sys_src, name) == _c_args(header, name), name
    for name in re.findall(r"pub fn (cg_[a-z0-9_]+)", sys_src):
        assert _rust_args(sys_src, name) == _c_args(header, name), name
