"""Host side of the boundary, without a GPU: the Op API's shape/type rules, the
native-compile step (template, md5 names, closure structs, c++ and hip
translation units), the runtime object model seen by closures, and the C++
interpreter -- exercised with small custom host-only ops, the way the
reference tests its own native-op plumbing (cgt/tests/test_multi_output.py,
cgt/tests/test_par_interp.py)."""
import ctypes
import os

import numpy as np
import pytest

from cgt_amd import compilation, core, rt
from cgt_amd.nn_ops import cross_channel_lrn as L
from cgt_amd.nn_ops import im2col as I
from cgt_amd.nn_ops import max_pool_2d as P


class FakeNode(object):
    """Stands in for a device node where only the shape is consulted."""

    def __init__(self, shape):
        self.shape = tuple(shape)
        self.typ = core.TensorType("f4", len(shape))
        self.value = self


@pytest.fixture(autouse=True)
def _fake_as_node(monkeypatch):
    orig = core.as_node
    monkeypatch.setattr(core, "as_node", lambda v: v if isinstance(v, FakeNode) else orig(v))


# ---------------------------------------------------------------- shape / type rules

def test_im2col_shape_rule():
    op = I.Im2Col(I.Im2ColInfo(11, 11, 0, 0, 4, 4))
    assert op.shp_apply([FakeNode((128, 3, 227, 227))]) == [128, 55, 55, 363]
    op = I.Im2Col(I.Im2ColInfo(3, 3, 1, 1, 2, 2))
    assert op.shp_apply([FakeNode((2, 3, 9, 11))]) == [2, 5, 6, 27]
    assert op.typ_apply([core.TensorType("f4", 4)]) == core.TensorType("f4", 4)


def test_max_pool_shape_rule_has_no_plus_one():
    # reference test_pool: (2,3,5,7), k=4, s=1 -> (2,3,1,3); demo shapes 28->13, 55->26, 56->27, 32->15
    assert P.MaxPool(P.PoolInfo(4, 4, 0, 0, 1, 1)).shp_apply([FakeNode((2, 3, 5, 7))])[0] == [2, 3, 1, 3]
    for H, k, s, want in [(28, 2, 2, 13), (55, 3, 2, 26), (56, 2, 2, 27), (32, 3, 2, 15)]:
        shp = P.MaxPool(P.PoolInfo(k, k, 0, 0, s, s)).shp_apply([FakeNode((1, 1, H, H))])
        assert shp == ([1, 1, want, want], [1, 1, want, want])
    typ = P.MaxPool(P.PoolInfo(2, 2, 0, 0, 2, 2)).typ_apply([core.TensorType("f4", 4)])
    assert typ == core.TupleType(core.TensorType("f4", 4), core.TensorType("i4", 4))


def test_mul22_shape_rule_all_variants():
    A, At, B, Bt = FakeNode((3, 5)), FakeNode((5, 3)), FakeNode((5, 7)), FakeNode((7, 5))
    assert core.Mul22(False, False).shp_apply([A, B]) == [3, 7]
    assert core.Mul22(False, True).shp_apply([A, Bt]) == [3, 7]
    assert core.Mul22(True, False).shp_apply([At, B]) == [3, 7]
    assert core.Mul22(True, True).shp_apply([At, Bt]) == [3, 7]
    assert core.BatchedMul22(False, False).shp_apply([FakeNode((2, 3, 5)), FakeNode((2, 5, 7))]) == [2, 3, 7]
    assert core.BatchedMul22(True, True).shp_apply([FakeNode((2, 5, 3)), FakeNode((2, 7, 5))]) == [2, 3, 7]


def test_available_impls_and_masks():
    ops = [I.Im2Col(I.Im2ColInfo(3, 3, 1, 1, 1, 1)), I.Col2Im(I.Im2ColInfo(3, 3, 1, 1, 1, 1)),
           P.MaxPool(P.PoolInfo(2, 2, 0, 0, 2, 2)), P.MaxPoolPullback(P.PoolInfo(2, 2, 0, 0, 2, 2)),
           L.CrossChannelLRNForward(L.LRNInfo(5, 1e-4, .75)), L.CrossChannelLRNBackward(L.LRNInfo(5, 1e-4, .75)),
           L.CrossChannelLRNTop(L.LRNInfo(5, 1e-4, .75)), L.CrossChannelLRNBackwardFromX(L.LRNInfo(5, 1e-4, .75)),
           core.Mul22(False, True), core.BatchedMul22(False, False)]
    for op in ops:
        assert "native_gpu" in op.available_impls and op.return_type == "byref"
    # Col2Im's four shape operands are host scalars: not dereferenced on the device
    T4, S = core.TensorType("f4", 4), core.TensorType("i8", 0)
    nci = ops[1].get_native_compile_info([T4, S, S, S, S], "gpu")
    assert nci.gpu_deref_mask == (True, False, False, False, False) and nci.involves_gpu()


# ---------------------------------------------------------------- native-compile step

def test_templated_code_and_names():
    triples = I.info2closure(I.Im2ColInfo(3, 3, 1, 1, 2, 2))
    code = compilation.gen_templated_code(["cgt_amd.h"], triples, "BODY")
    assert code.startswith('#include "cgt_common.h"\n#include "cgt_amd.h"\ntypedef struct $closure {\nint kernel_h;')
    assert code.endswith("} $closure;\nBODY")
    h1 = compilation.hash_seq(code, "flags", "1")
    assert h1 == compilation.hash_seq(code, "flags", "1") and h1 != compilation.hash_seq(code, "flags", "2")
    assert compilation._funcname(h1) == "call_" + h1 and len(h1) == 32


def test_closure_struct_layouts():
    conv = compilation._build_closure(I.info2closure(I.Im2ColInfo(11, 12, 1, 2, 4, 5)))
    assert ctypes.sizeof(conv) == 24      # six ints, as the reference's conv_closure (pooling.h:7-14)
    assert (conv.kernel_h, conv.kernel_w, conv.pad_h, conv.pad_w, conv.stride_h, conv.stride_w) == (11, 12, 1, 2, 4, 5)
    lrn = compilation._build_closure(L.make_closure(L.LRNInfo(5, 1e-4, 0.75), 2.0))
    assert ctypes.sizeof(lrn) == 32 and lrn.localsize == 5 and lrn.k == 2.0
    mm = compilation._build_closure(core.Mul22(True, False).get_closure())
    assert ctypes.sizeof(mm) == 16 and mm.tA and not mm.tB


def test_prebuild_standard_ops_exports_call_symbols():
    built = compilation.prebuild_standard_ops()
    assert len(built) == 34
    for c in built:
        assert c.fptr_address and c.return_type in ("byref", "byval") and c.kind == "native"
    assert [c.return_type for c in built].count("byval") == 2
    cache = compilation.get_compile_info()["CACHE_ROOT"]
    assert any(f.endswith(".so") for f in os.listdir(cache))


class AddHostOp(core.Op):
    """z = x + y on int64 host arrays plus the sum, as a tuple: a host-only op."""
    available_impls = ("native_cpu",)

    def get_native_compile_info(self, input_types, devtype):
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtTuple* write) {
                cgtArray *x = reads[0], *y = reads[1];
                cgtArray* z = static_cast<cgtArray*>(write->getitem(0));
                cgtArray* total = static_cast<cgtArray*>(write->getitem(1));
                cgt_check(x->size() == y->size() && z->size() == x->size(), "size mismatch %ld %ld", x->size(), y->size());
                if (cgtGlobalStatus != cgtStatusOK) return;
                long s = 0;
                for (long i = 0; i < x->size(); ++i) { z->at<long>(i) = x->at<long>(i) + y->at<long>(i) + cl->bias; s += z->at<long>(i); }
                total->at<long>(0) = s;
                cgt_assert(x->ndim() == 2 && x->stride(0) == x->shape()[1] && x->stride(1) == 1);
                cgt_assert(x->devtype() == cgtCPU && x->dtype() == cgt_i8 && !x->ownsdata());
            }"""
        return core.NativeCompileInfo(code, closure_triples=[("bias", ctypes.c_long, 7)])


def _compile(op, types):
    nci = op.get_native_compile_info(types, "cpu")
    nci.op_str, nci.return_type, nci.n_in = str(op), "byref", len(types)
    return compilation.nci2callable(nci)


def test_custom_host_op_tuple_output_and_error_status():
    T = core.TensorType("i8", 2)
    call = _compile(AddHostOp(), [T, T])
    x = np.arange(6, dtype=np.int64).reshape(2, 3)
    y = 10 * np.ones((2, 3), np.int64)
    z, total = np.zeros((2, 3), np.int64), np.zeros((), np.int64)
    call.call([x, y], (z, total))
    assert np.array_equal(z, x + y + 7) and int(total) == int((x + y + 7).sum())
    # a failing cgt_check surfaces as an exception on the host
    from cgt_amd.capi import CgtAmdError
    with pytest.raises(CgtAmdError, match="size mismatch"):
        call.call([x, np.ones((5, 1), np.int64)], (z, total))
    call.call([x, y], (z, total))   # status was cleared


def test_hip_translation_unit_compiles_and_links():
    # a two-translation-unit op: host closure + device launcher, as the
    # reference shapes its CUDA ops (cross_channel_lrn.py:24-55)
    hip = r"""
        #include <hip/hip_runtime.h>
        __global__ void scale_kernel_$function(float* x, float a, long n) {
            long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
            if (i < n) x[i] *= a;
        }
        void launchker_$function(float* x, float a, long n, void* stream) {
            scale_kernel_$function<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(x, a, n);
        }"""
    code = r"""
        extern void launchker_$function(float* x, float a, long n, void* stream);
        CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
            launchker_$function((float*)write->data(), cl->a, write->size(), cgt_get_stream());
        }"""
    nci = core.NativeCompileInfo(code, closure_triples=[("a", ctypes.c_float, 2.0)],
                                 extra_srcs=[core.SrcFile("hip", hip)], gpu_deref_mask=(True,))
    nci.op_str, nci.return_type, nci.n_in = "scale", "byref", 1
    call = compilation.nci2callable(nci)
    assert call.fptr_address
    with pytest.raises(NotImplementedError):
        compilation.TranslationUnit([core.SrcFile("cuda", "")], "").compile("x", "/tmp/x.so")


# ---------------------------------------------------------------- runtime objects and interpreter

def test_runtime_objects_roundtrip():
    lib = rt.lib()
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    o = rt.to_cgt(x)
    assert lib.cgt_rt_kind(o.handle) == rt.ARRAY_KIND
    assert lib.cgt_rt_array_ndim(o.handle) == 2 and lib.cgt_rt_array_dtype(o.handle) == 11
    assert lib.cgt_rt_array_stride(o.handle, 0) == 4 and lib.cgt_rt_array_nbytes(o.handle) == 48
    assert lib.cgt_rt_array_data(o.handle) == x.ctypes.data      # a view, not a copy
    t = rt.to_cgt((x, 5))
    assert lib.cgt_rt_kind(t.handle) == rt.TUPLE_KIND and lib.cgt_rt_tuple_len(t.handle) == 2
    back = rt.from_cgt_handle(t.handle)
    assert np.array_equal(back[0], x) and int(back[1]) == 5
    own = rt.CgtObject(lib.cgt_rt_array_new(2, (ctypes.c_long * 2)(3, 4), 11, rt.CPU))
    assert lib.cgt_rt_copy_object(own.handle, o.handle) == 0
    assert np.array_equal(rt.from_cgt_handle(own.handle), x)


def test_interpreter_alloc_reuse_and_byref():
    T = core.TensorType("i8", 2)
    call = _compile(AddHostOp(), [T, T])
    it = rt.Interpreter(8)
    cpu = rt.CPU
    it.load_argument(0, (0, cpu))
    it.load_argument(1, (1, cpu))
    it.set_slot(2, 2)             # shape scalars live in slots, on the host
    it.set_slot(3, 3)
    it.alloc(np.int64, [(2, cpu), (3, cpu)], (4, cpu))
    it.alloc(np.int64, [], (5, cpu))
    it.build_tup([(4, cpu), (5, cpu)], (6, cpu))
    it.return_byref(call, [(0, cpu), (1, cpu)], (6, cpu))
    x = np.arange(6, dtype=np.int64).reshape(2, 3)
    y = np.ones((2, 3), np.int64)
    it.run([x, y])
    z, total = it.get_array(6)
    assert np.array_equal(z, x + y + 7) and int(total) == int((x + y + 7).sum())
    p1 = rt.lib().cgt_rt_array_data(rt.lib().cgt_rt_interp_get_slot(it.handle, 4))
    it.run([x + 1, y])
    p2 = rt.lib().cgt_rt_array_data(rt.lib().cgt_rt_interp_get_slot(it.handle, 4))
    assert p1 == p2, "Alloc must reuse the output buffer while the shape is unchanged"
    assert np.array_equal(it.get_array(6)[0], x + 1 + y + 7)
    with pytest.raises(ValueError):
        it.alloc(np.int64, [], (99, cpu))


def test_shape_int_keeps_its_expression():
    from cgt_amd.core import ShapeInt, ceil_divide, shape_depends_on
    leaf = object()
    H = ShapeInt(28, ("size", leaf, 2))
    m = (H + 2 * 1 - 3) // 1 + 1
    assert m == 28 and isinstance(m, ShapeInt) and shape_depends_on(m.expr) == [leaf]
    p = ceil_divide(m + 2 * 0 - 2, 2)
    assert p == 13 and p.expr[0] == "ceildiv"
    assert (ShapeInt(3) * 4).is_constant() and (3 * H).expr == ("*", ("const", 3), ("size", leaf, 2))
    assert (-H).expr == ("neg", ("size", leaf, 2)) and (10 - H) == -18 and (H - 10).expr[0] == "-"
    assert int(H) + 1 == 29 and type(int(H)) is int and [0] * ShapeInt(2) == [0, 0]
    from cgt_amd.function import _eval_expr
    assert _eval_expr(("ceildiv", ("const", -3), ("const", 2))) == 0
    assert _eval_expr(("//", ("const", -3), ("const", 2))) == -2


def test_interpreter_shape_instructions_and_alloc_capacity():
    # Size / integer-op closures of the runtime computing an Alloc's shape from the argument
    # at every run; a buffer that has grown serves the smaller shapes after it
    from cgt_amd.function import _IntOpClosure, _RtCallable, _SizeClosure
    it = rt.Interpreter(8)
    cpu = rt.CPU
    it.load_argument(0, (0, cpu))
    it.set_slot(1, 3)
    it.set_slot(2, 2)
    it.return_byval(_RtCallable("cgt_rt_op_size", _SizeClosure(0)), [(0, cpu)], (3, cpu))
    it.return_byval(_RtCallable("cgt_rt_op_intop", _IntOpClosure(2)), [(3, cpu), (1, cpu)], (4, cpu))     # 3 * n
    it.return_byval(_RtCallable("cgt_rt_op_intop", _IntOpClosure(4)), [(3, cpu), (2, cpu)], (5, cpu))     # ceil(n / 2)
    it.return_byval(_RtCallable("cgt_rt_op_intop", _IntOpClosure(3)), [(3, cpu), (2, cpu)], (6, cpu))     # n // 2
    it.alloc(np.float32, [(4, cpu), (5, cpu)], (7, cpu))
    L = rt.lib()

    def run(n):
        it.run([np.zeros((n, 2), np.int64)])
        h = L.cgt_rt_interp_get_slot(it.handle, 7)
        shp = L.cgt_rt_array_shape(h)
        return (shp[0], shp[1]), L.cgt_rt_array_data(h), int(it.get_array(6))
    s5, p5, f5 = run(5)
    assert s5 == (15, 3) and f5 == 2
    s5b, p5b, _ = run(5)
    assert p5b == p5
    s9, p9, f9 = run(9)
    assert s9 == (27, 5) and f9 == 4
    s4, p4, _ = run(4)
    assert s4 == (12, 2) and p4 == p9, "a shape that fits the grown buffer must not allocate"


# ---------------------------------------------------------------- conv-layer glue ops (host logic only)

def test_elwise_binary_type_rules():
    # reference core.py:1319-1333: 'p' promotes, 'f' gives floatX, comparisons give i1;
    # the output takes the rank of the non-scalar operand
    F4, B4, F0 = core.TensorType("f4", 4), core.TensorType("i1", 4), core.TensorType("f4", 0)
    assert core.ElwiseBinary("*", (False, False)).typ_apply([F4, B4]) == F4
    assert core.ElwiseBinary("*", (False, False)).typ_apply([B4, B4]) == B4
    assert core.ElwiseBinary("/", (False, False)).typ_apply([B4, B4]) == F4
    assert core.ElwiseBinary(">=", (False, True)).typ_apply([F4, F0]) == B4
    assert core.ElwiseBinary("+", (True, False)).typ_apply([F0, F4]) == F4
    with pytest.raises(AssertionError):
        core.ElwiseBinary("+", (False, False)).typ_apply([F4, F0])       # mask must match the ranks
    assert core.ElwiseBinary("<", (False, False)).get_diff(2) == [False, False]
    assert core.ElwiseBinary("-", (False, False)).get_diff(2) == [True, True]


def test_glue_closures_and_hashes():
    # one compiled library per op class: the op code / axes / value travel in the closure
    a, b = core.ElwiseBinary("+", (False, False)), core.ElwiseBinary("*", (False, True))
    assert a.get_hash() != b.get_hash()
    ca = a.get_native_compile_info([core.TensorType("f4", 2)] * 2, "gpu")
    cb = b.get_native_compile_info([core.TensorType("f4", 2), core.TensorType("f4", 0)], "gpu")
    assert ca.func_code == cb.func_code and ca.gpu_deref_mask == (True, True)
    assert [t[2] for t in b.get_closure()] == [core.BINARY_CODES.index("*"), 0, 1]
    assert core.Repeat((0, 2, 3)).get_closure()[0][2] == 0b1101
    assert core.Sum((1,)).get_closure()[0][2] == 0b10
    S = core.TensorType("i8", 0)
    nci = core.Repeat((0, 2, 3)).get_native_compile_info([core.TensorType("f4", 4), S, S, S], "gpu")
    assert nci.gpu_deref_mask == (True, False, False, False)        # repeat counts stay on the host
    assert core.Fill(2.0).typ_apply([S, S, S]) == core.TensorType("f4", 3)
    assert core.ElwiseUnary("sign").get_diff(1) == [False] and core.ElwiseUnary("tanh").get_diff(1) == [True]
    # op codes agree with the C header
    hdr = open(os.path.join(os.path.dirname(__file__), "..", "include", "cgt_amd.h")).read()
    for i, name in enumerate(["MUL", "ADD", "SUB", "DIV", "LT", "GT", "LE", "GE", "POW", "EQ", "NE"]):
        assert "#define CGT_AMD_BIN_%s %d\n" % (name, i) in hdr
    for i, name in enumerate(["ABS", "COS", "EXP", "LOG", "NEG", "SIGN", "SIN", "SQUARE", "SQRT", "TANH", "SIGMOID"]):
        assert "#define CGT_AMD_UN_%s %d\n" % (name, i) in hdr
