"""The reference-side adapter (tinytensor_amd/host/adapter/.../backend_amd.{h,cpp}) against the reference's interface.

The adapter derives from tinytensor::BackendBase, which this image's toolchain cannot build the library around, so the
adapter is checked mechanically instead (CPU only, and only where the reference tree is present):
  1. every pure virtual of tinytensor/tensor/backend_base.h has an override in backend_amd.h with the same signature
     string (name, parameter list with parameter names, qualifiers, return type), and nothing else is overridden;
  2. every override has exactly one definition in backend_amd.cpp with the same parameter types;
  3. the class is concrete: backend_amd.cpp and an instantiation compile (syntax only) against the reference's own
     backend_base.h and storage_base.h, with a few lines of stand-in declarations for the <tt/...> headers that need
     a newer standard library than this image has.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference"
BASE_H = os.path.join(REFERENCE, "tinytensor", "tensor", "backend_base.h")
ADAPTER = os.path.join(ROOT, "tinytensor_amd", "host", "adapter", "tinytensor")
AMD_H = os.path.join(ADAPTER, "tensor", "backend", "amd", "backend_amd.h")
AMD_CPP = os.path.join(ADAPTER, "tensor", "backend", "amd", "backend_amd.cpp")

pytestmark = pytest.mark.skipif(not os.path.exists(BASE_H) or shutil.which("g++") is None,
                                reason="needs the reference tree and g++")


def _squash(text: str) -> str:
    text = re.sub(r"\s+", " ", text).strip()
    text = re.sub(r"\(\s+", "(", text)
    text = re.sub(r"\s+\)", ")", text)
    text = re.sub(r"\s*,\s*", ", ", text)
    return text


def _strip_comments(text: str) -> str:
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def base_pure_virtuals():
    """Signature strings of the pure virtuals: `auto name(params) const -> R` / `void name(params) const`."""
    text = _strip_comments(open(BASE_H).read())
    body = text[text.index("class BackendBase"):]
    out = []
    for stmt in body.split(";"):
        if "virtual" not in stmt or not re.search(r"=\s*0\s*$", stmt):
            continue
        s = stmt.replace("[[nodiscard]]", " ")
        s = re.sub(r"\bvirtual\b", " ", s)
        s = re.sub(r"=\s*0\s*$", "", s)
        out.append(_squash(s))
    return out


def _preprocess(*paths):
    """The files' own macros expanded, with no header pulled in."""
    src = ""
    for p in paths:
        src += "\n".join(l for l in open(p).read().splitlines() if not l.lstrip().startswith("#include")) + "\n"
    proc = subprocess.run(["g++", "-E", "-P", "-x", "c++", "-std=c++20", "-"], input=src, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return proc.stdout


def adapter_overrides():
    text = _preprocess(AMD_H)
    body = text[text.index("class BackendAMD"):]
    body = body[body.index("{") + 1:]
    out = []
    for stmt in body.split(";"):
        if not re.search(r"\boverride\s*$", stmt):
            continue
        s = stmt.replace("[[nodiscard]]", " ")
        s = re.sub(r"\bpublic\s*:", " ", s)
        s = re.sub(r"\boverride\s*$", "", s)
        out.append(_squash(s))
    return out


def _split_params(params: str):
    parts, depth, cur = [], 0, ""
    for ch in params:
        if ch in "<(":
            depth += 1
        elif ch in ">)":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        parts.append(cur)
    return [p.strip() for p in parts]


def _types_only(params: str) -> str:
    """The parameter list with parameter names removed."""
    out = []
    for p in _split_params(params):
        m = re.match(r"^(.*?[&*\s])([A-Za-z_]\w*)$", p)
        if m and re.search(r"[&*]|\w\s", m.group(1)):
            p = m.group(1)
        out.append(re.sub(r"\s+", " ", p).strip().replace(" &", "&").replace("& ", "&"))
    return ", ".join(out)


def _key(signature: str):
    m = re.match(r"^(?:auto|void)\s+(\w+)\((.*)\)\s*const(?:\s*->\s*(.*))?$", signature)
    assert m, signature
    return m.group(1), _types_only(m.group(2)), (m.group(3) or "void").strip()


def test_every_pure_virtual_is_overridden_with_an_identical_signature():
    base = base_pure_virtuals()
    mine = adapter_overrides()
    assert len(base) == open(BASE_H).read().count("= 0;") and len(base) > 200  # every pure virtual was parsed
    assert len(set(base)) == len(base) and len(set(mine)) == len(mine)
    missing = sorted(set(base) - set(mine))
    extra = sorted(set(mine) - set(base))
    assert not missing, f"pure virtuals of backend_base.h without an identical override: {missing[:8]}"
    assert not extra, f"overrides that match no pure virtual of backend_base.h: {extra[:8]}"


def test_every_override_has_exactly_one_definition():
    declared = sorted(_key(s) for s in adapter_overrides())
    text = _preprocess(AMD_H, AMD_CPP)
    text = text[text.index("class BackendAMD"):]
    text = text[text.index("};"):]                           # past the class: the definitions
    found = []
    for m in re.finditer(r"\b(?:auto|void)\s+BackendAMD::(\w+)\(([^{;]*?)\)\s*const(?:\s*->\s*([^{;]*?))?\s*\{", text, flags=re.S):
        found.append((m.group(1), _types_only(_squash(m.group(2))), _squash(m.group(3) or "void")))
    found.sort()
    assert len(found) == len(set(found)), "a member is defined twice"
    # one const member beside the overrides: the two products of a matmul's backward in one call, no virtual of BackendBase
    extra = [f for f in found if f not in declared]
    assert extra == [("batched_matmul_pair", "const Tensor&, const Tensor&, const Tensor&, const Tensor&", "std::pair<Tensor, Tensor>")], extra
    found = [f for f in found if f not in extra]
    assert found == declared, (sorted(set(declared) - set(found))[:6], sorted(set(found) - set(declared))[:6])


def test_not_implemented_operations_say_so():
    text = _preprocess(AMD_H, AMD_CPP)
    assert text.count("not_implemented(") > 100              # every operation off the GEMM path answers with a TTException
    assert '" is not implemented on the AMD device"' in open(AMD_CPP).read()


# Stand-ins for the few declarations of <tt/...> that backend_base.h and the adapter use.  The real headers need
# <format> and constexpr std::string (libstdc++ 13); these lines only declare names, they implement nothing.
STUBS = {
    "tt/exception.h": """#pragma once
#include <cstdlib>
#include <exception>
#include <iostream>
#include <string>
namespace tinytensor {
class TTException : public std::exception {
public:
    TTException(const std::string &m, const char *, const char *, int) : message(m) {}
    const char *what() const noexcept override { return message.c_str(); }
    std::string message;
};
}
#define TT_EXCEPTION(msg) throw tinytensor::TTException(msg, __FILE__, __PRETTY_FUNCTION__, __LINE__)
#define TT_ERROR(msg) { std::cout << msg << std::endl; std::exit(1); }
""",
    "tt/device.h": """#pragma once
namespace tinytensor {
enum class Backend { cpu, amd };
struct Device { Backend backend; int id; };
constexpr Device kCPU = Device{Backend::cpu, 0};
}
""",
    "tt/scalar.h": """#pragma once
#include <cstdint>
namespace tinytensor {
enum class ScalarType { bool8, u8, i16, i32, i64, f32, f64 };
constexpr ScalarType kBool = ScalarType::bool8, kU8 = ScalarType::u8, kI16 = ScalarType::i16, kI32 = ScalarType::i32,
                     kI64 = ScalarType::i64, kF32 = ScalarType::f32, kF64 = ScalarType::f64, kDefaultFloat = ScalarType::f32;
constexpr bool is_float_dtype(ScalarType t) { return t == kF32 || t == kF64; }
class Scalar {
public:
    template <typename T> explicit Scalar(T v);
    ScalarType dtype() const;
    template <typename T> T to() const;
};
}
""",
    "tt/shape.h": """#pragma once
#include <initializer_list>
#include <vector>
namespace tinytensor {
class Shape {
public:
    Shape(std::initializer_list<int> d);
    int numel() const noexcept;
    int ndim() const noexcept;
    int &operator[](int i);
    int operator[](int i) const;
    const std::vector<int> &to_vec() const;
};
}
""",
    "tt/random.h": """#pragma once
#include <cstdint>
namespace tinytensor {
class Generator { public: uint64_t operator()() noexcept; };
}
""",
    "tt/tensor.h": """#pragma once
#include <memory>
#include <ostream>
#include <tt/device.h>
#include <tt/scalar.h>
#include <tt/shape.h>
namespace tinytensor {
class StorageBase;
class Tensor {
public:
    Tensor(std::shared_ptr<StorageBase> storage, ScalarType dtype, Shape shape, Device device);
    ScalarType dtype() const; Device device() const; int offset() const;
    const Shape &shape() const; const Shape &stride() const;
    int numel() const; int size(int) const; Tensor contiguous() const; Tensor to(Device) const;
    template <typename T> T &get_storage() const;
    friend std::ostream &operator<<(std::ostream &os, const Tensor &);
};
}
""",
}


def test_adapter_is_concrete_against_the_reference_interface(tmp_path):
    for name, text in STUBS.items():
        path = tmp_path / name
        path.parent.mkdir(parents=True, exist_ok=True)
        path.write_text(text)
    (tmp_path / "instantiate.cpp").write_text(
        '#include "tensor/backend/amd/backend_amd.h"\n#include <memory>\n'
        "auto make() { return std::make_unique<tinytensor::amd::BackendAMD>(); }\n")
    flags = ["g++", "-std=c++20", "-fsyntax-only", "-I", str(tmp_path), "-I", os.path.join(REFERENCE, "tinytensor"),
             "-I", os.path.join(ROOT, "include"), "-I", ADAPTER]
    for src in (str(tmp_path / "instantiate.cpp"), AMD_CPP):
        proc = subprocess.run(flags + [src], capture_output=True, text=True)
        assert proc.returncode == 0, proc.stderr[-3000:]
