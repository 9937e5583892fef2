"""The native-compile step: NativeCompileInfo -> shared library -> NativeCallable.

Follows the reference's cgt/compilation.py:521-749: the op's code is wrapped
with `#include "cgt_common.h"`, its includes and a `typedef struct $closure`
generated from the closure triples; $function / $closure / $setup / $teardown
are renamed with an md5 over (templated code, compiler flags, ABI version, the
text of the headers every closure includes, extra sources); each source file is compiled (`c++` for "c++", `hipcc
--offload-arch=gfx950` for "hip" -- the reference's "cuda"/nvcc slot), linked
into <cache>/<md5>.so, loaded with ctypes, and the closure struct is built as
a ctypes.Structure.  A library that is already in the cache is not rebuilt.
"""
import ctypes
import hashlib
import os
import string
import subprocess
import sys

from . import build as _build
from . import core, rt

# bump when the object model in csrc/include/cgt_common.h changes layout
CPP_ABI_VERSION = 2
# headers every closure is compiled against: cgtArray's accessors are inline, so
# their text is part of each cached library and therefore of its cache key
_ABI_HEADERS = ("cgt_common.h", "cgt_amd.h")
_abi_headers_hash = None

_COMPILE_CONFIG = None
_LIBRARIES = {}
_struct_cache = {}

_ctypes2str = {
    ctypes.c_byte: "uint8_t",
    ctypes.c_bool: "bool",
    ctypes.c_char: "char",
    ctypes.c_int: "int",
    ctypes.c_long: "long",
    ctypes.c_void_p: "void*",
    ctypes.c_double: "double",
    ctypes.c_float: "float",
}


def get_compile_info():
    global _COMPILE_CONFIG
    if _COMPILE_CONFIG is None:
        cache = os.environ.get("CGT_AMD_CACHE_DIR", os.path.join(_build.HERE, "_cache"))
        os.makedirs(cache, exist_ok=True)
        includes = "-I%s -I%s -I/opt/rocm/include" % (_build.RT_INCLUDE, _build.INCLUDE)
        debug = os.environ.get("CGT_AMD_DEBUG_CPP", "0") == "1"
        cpp_flags = "-fvisibility=hidden -std=c++11 -fPIC" + (" -O0 -g" if debug else " -O3 -DNDEBUG")
        hip_flags = ("--offload-arch=%s -std=c++17 -fPIC -fvisibility=hidden -O3 "
                     "-Xclang -target-feature -Xclang -packed-fp32-ops -Wno-unused-command-line-argument" % _build.ARCH)
        link_flags = "-L%s -lcgt_rt -lcgt_amd -Wl,-rpath,%s -shared -rdynamic" % (_build.LIBDIR, _build.LIBDIR)
        _COMPILE_CONFIG = dict(CACHE_ROOT=cache, INCLUDES=includes, CPP_FLAGS=cpp_flags, HIP_FLAGS=hip_flags,
                               LINK_FLAGS=link_flags, CXX=_build.CXX, HIPCC=_build.HIPCC,
                               HIP_LINK_FLAGS="-L/opt/rocm/lib -lamdhip64")
    return _COMPILE_CONFIG


def abi_headers_hash():
    """md5 over the text of the headers the closures include."""
    global _abi_headers_hash
    if _abi_headers_hash is None:
        h = hashlib.md5()
        for name in _ABI_HEADERS:
            for d in (_build.RT_INCLUDE, _build.INCLUDE):
                path = os.path.join(d, name)
                if os.path.exists(path):
                    with open(path, "rb") as fh:
                        h.update(fh.read())
                    break
            else:
                raise RuntimeError("header %s not found" % name)
        _abi_headers_hash = h.hexdigest()
    return _abi_headers_hash


def hash_seq(*strings):
    h = hashlib.md5()
    for s in strings:
        h.update(s.encode("utf-8"))
        h.update(b"\0")
    return h.hexdigest()


def _funcname(prefix):
    return "call_" + prefix


def _setupname(prefix):
    return "setup_" + prefix


def _teardownname(prefix):
    return "teardown_" + prefix


def _closurename(prefix):
    return "closure_" + prefix


def gen_struct_code(triples):
    if triples is None:
        return ""
    lines = ["typedef struct $closure {"]
    for (fieldname, fieldtype, _val) in triples:
        lines.append("%s %s;" % (_ctypes2str[fieldtype], fieldname))
    lines.append("} $closure;")
    return "\n".join(lines) + "\n"


def gen_templated_code(includes, closure_info, func_code):
    out = []
    for fname in ["cgt_common.h"] + list(includes):
        out.append('#include "%s"' % fname)
    return "\n".join(out) + "\n" + gen_struct_code(closure_info) + func_code


def _build_closure(triples):
    if triples is None:
        return None
    fields = [(name, typ) for (name, typ, _val) in triples]
    key = tuple((n, t.__name__) for n, t in fields)
    S = _struct_cache.get(key)
    if S is None:
        S = type("Closure", (ctypes.Structure,), {"_fields_": fields})
        _struct_cache[key] = S
    return S(*[val for (_n, _t, val) in triples])


def get_or_load_lib(libname):
    if libname not in _LIBRARIES:
        rt.lib()  # the closures link against libcgt_rt / libcgt_amd
        _LIBRARIES[libname] = ctypes.cdll.LoadLibrary(libname)
    return _LIBRARIES[libname]


class TranslationUnit(object):
    """All the input that goes into building the native binary of one op."""

    def __init__(self, srcfiles, link_flags):
        self.srcfiles = srcfiles
        self.link_flags = link_flags

    def compile(self, prefix, libpath):
        d = get_compile_info()
        cache = d["CACHE_ROOT"]
        cmds, objs = [], []
        uses_hip = False
        for i, (lang, code) in enumerate(self.srcfiles):
            if lang == "c++":
                srcpath = os.path.join(cache, "%s_%d.cpp" % (prefix, i))
                cmds.append("%s %s %s -c -o %s.o %s" % (d["CXX"], d["CPP_FLAGS"], srcpath, srcpath, d["INCLUDES"]))
            elif lang == "hip":
                srcpath = os.path.join(cache, "%s_%d.hip" % (prefix, i))
                cmds.append("%s %s %s -c -o %s.o %s" % (d["HIPCC"], d["HIP_FLAGS"], srcpath, srcpath, d["INCLUDES"]))
                uses_hip = True
            else:
                raise NotImplementedError("source language %r (this build compiles c++ and hip)" % lang)
            with open(srcpath, "w") as fh:
                fh.write(code)
            objs.append(srcpath + ".o")
        tmp = libpath + ".tmp.%d" % os.getpid()
        linker = d["HIPCC"] + " --offload-arch=" + _build.ARCH if uses_hip else d["CXX"] + " " + d["CPP_FLAGS"]
        cmds.append("%s %s %s %s -o %s" % (linker, " ".join(objs), d["LINK_FLAGS"], self.link_flags, tmp))
        bigcmd = " && ".join(cmds)
        if os.environ.get("CGT_AMD_VERBOSE", "0") == "1":
            print("\x1b[32m%s\x1b[0m" % bigcmd, file=sys.stderr)
        proc = subprocess.run(bigcmd, shell=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("native compile failed:\n%s\n%s" % (bigcmd, proc.stdout))
        os.replace(tmp, libpath)


def nci2callable(nci):
    template_code = gen_templated_code(nci.includes, nci.closure_triples, nci.func_code)
    d = get_compile_info()
    prefix = hash_seq(template_code, d["CPP_FLAGS"], str(CPP_ABI_VERSION), abi_headers_hash(),
                      *(src.code for src in nci.extra_srcs))
    names = dict(function=_funcname(prefix), closure=_closurename(prefix), setup=_setupname(prefix),
                 teardown=_teardownname(prefix))
    srcfiles = [core.SrcFile("c++", string.Template(template_code).substitute(names))]
    srcfiles.extend(core.SrcFile(sf.lang, string.Template(sf.code).substitute(names)) for sf in nci.extra_srcs)
    libpath = os.path.join(d["CACHE_ROOT"], prefix + ".so")
    if not os.path.exists(libpath):
        TranslationUnit(srcfiles, nci.link_flags).compile(prefix, libpath)
    lib = get_or_load_lib(libpath)
    fptr = getattr(lib, _funcname(prefix))
    fptr.restype = None
    setup_fptr = getattr(lib, _setupname(prefix)) if nci.setup else None
    teardown_fptr = getattr(lib, _teardownname(prefix)) if nci.teardown else None
    cldata = _build_closure(nci.closure_triples)
    return core.NativeCallable(nci.n_in, nci.return_type, nci.op_str, fptr, cldata=cldata,
                               setup_fptr=setup_fptr, teardown_fptr=teardown_fptr,
                               store_objects=nci.store_objects)


def prebuild_standard_ops():
    """Compile the closures of every hot-path op into the cache (no GPU needed):
    one library per op type, since geometry travels in the closure struct."""
    from . import nn_ops
    T4 = core.TensorType("f4", 4)
    T3 = core.TensorType("f4", 3)
    T2 = core.TensorType("f4", 2)
    I4 = core.TensorType("i4", 4)
    S = core.TensorType("i8", 0)
    info = nn_ops.im2col.Im2ColInfo(3, 3, 1, 1, 1, 1)
    pinfo = nn_ops.max_pool_2d.PoolInfo(2, 2, 0, 0, 2, 2)
    linfo = nn_ops.cross_channel_lrn.LRNInfo(5, 1e-4, 0.75)
    cinfo = nn_ops.conv_same.ConvSameInfo(3, 3)
    T1 = core.TensorType("f4", 1)
    todo = [
        (nn_ops.im2col.Im2Col(info), [T4]),
        (nn_ops.im2col.Col2Im(info), [T4, S, S, S, S]),
        (nn_ops.max_pool_2d.MaxPool(pinfo), [T4]),
        (nn_ops.max_pool_2d.MaxPoolPullback(pinfo), [T4, T4, I4, T4]),
        (nn_ops.cross_channel_lrn.CrossChannelLRNForward(linfo), [T4]),
        (nn_ops.cross_channel_lrn.CrossChannelLRNBackward(linfo), [T4, T4, T4, T4]),
        (nn_ops.cross_channel_lrn.CrossChannelLRNTop(linfo), [T4]),
        (nn_ops.cross_channel_lrn.CrossChannelLRNBackwardFromX(linfo), [T4, T4]),
        (core.Mul22(False, True), [T2, T2]),
        (core.BatchedMul22(False, False), [T3, T3]),
        (core.Transpose((0, 3, 1, 2)), [T4]),
        (nn_ops.conv_same.ConvPad(cinfo), [T4]),
        (nn_ops.conv_same.ConvForward(cinfo), [T4, T1, T4]),
        (nn_ops.conv_same.ConvForward(cinfo, True, True), [T4, T1, T4, T4]),
        (nn_ops.conv_same.ConvBackwardData(cinfo), [T1, T4, T4]),
        (nn_ops.conv_same.ConvBackwardFilter(cinfo), [T1, T1, T4, T4]),
        (nn_ops.conv_same.ConvPadPoolPullback(cinfo, pinfo), [T4, T4, I4, T4]),
        (nn_ops.conv_col.ConvColForward(), [T4, T4]),
        (nn_ops.conv_col.ConvColForward(True, True), [T4, T4, T4]),
        (nn_ops.conv_col.ConvColBackwardData(), [T4, T4, T4]),
        (nn_ops.conv_col.ConvColBackwardFilter(), [T4, T4, T4]),
        (nn_ops.conv_col.ConvPatchForward(info), [T4, T4]),
        (nn_ops.conv_col.ConvPatchForward(info, True, True), [T4, T4, T4]),
        (nn_ops.conv_col.ConvPatchBackwardData(info), [T4, T4, T4]),
        (nn_ops.conv_col.ConvPatchBackwardFilter(info), [T4, T4, T4]),
        (core.Transport("gpu"), [T4]),
        # conv-layer glue: the closure code is generic over element type and
        # rank, so one library per op class serves every use
        (core.ElwiseUnary("exp"), [T4]),
        (core.ElwiseBinary("+", (False, False)), [T4, T4]),
        (core.Repeat((0, 2, 3)), [T4, S, S, S]),
        (core.Sum((0, 2, 3)), [T4]),
        (core.Fill(0.0), [S, S, S, S]),
        (core.ExtentAsFloat(), [S]),
        # by-value closures a compiled `function` replays
        (core.Reshape(), [T4, S, S]),
        (core.TupleIndex(0), [core.TupleType(T4, I4)]),
    ]
    built = []
    for op, types in todo:
        nci = op.get_native_compile_info(types, "gpu")
        nci.op_str, nci.return_type, nci.n_in = str(op), op.return_type, len(types)
        built.append(nci2callable(nci))
    return built
