// libcgt_rt: host runtime behind compiled op closures -- the cgtArray /
// cgtTuple object model, memory management that sends cgtGPU traffic to
// libcgt_amd (HIP), a C API the Python host uses to build objects and fire
// closures, and a sequential instruction interpreter that replays a fixed
// list of Alloc / BuildTup / ReturnByRef / ReturnByVal instructions without
// Python in the loop.
//
// Plays the part of the reference's src/cgt_common.cpp (objects, cgt_alloc /
// cgt_free / cgt_memcpy), of the object-conversion and apply_byref parts of
// src/cycgt.pyx, and of the SequentialInterpreter of src/execution.cpp.
#include "cgt_common.h"
#include "cgt_amd.h"

#include <cstring>
#include <string>
#include <vector>

// ------------------------------------------------------------------ status

extern "C" {
cgtStatus cgtGlobalStatus = cgtStatusOK;
char cgtGlobalErrorMsg[1000] = "";
static void* g_stream = NULL;
void* cgt_get_stream(void) { return g_stream; }
void cgt_set_stream(void* s) { g_stream = s; }
}

// ------------------------------------------------------------------ memory

void* cgt_alloc(cgtDevtype devtype, long nbytes) {
    if (devtype == cgtCPU) return malloc(nbytes > 0 ? (size_t)nbytes : 1);
    void* p = cgt_amd_alloc(nbytes);
    cgt_check(p != NULL, "cgt_alloc(GPU, %ld): %s", nbytes, cgt_amd_last_error());
    return p;
}

void cgt_free(cgtDevtype devtype, void* ptr) {
    if (devtype == cgtCPU) free(ptr);
    else cgt_check(cgt_amd_free(ptr) == CGT_AMD_OK, "cgt_free(GPU): %s", cgt_amd_last_error());
}

void cgt_memcpy(cgtDevtype dest, cgtDevtype src, void* dest_ptr, void* src_ptr, long nbytes) {
    if (dest == cgtCPU && src == cgtCPU) {
        memcpy(dest_ptr, src_ptr, (size_t)nbytes);
        return;
    }
    // device to device: ordered on the stream the closures launch on, no host wait
    int rc = (dest == cgtGPU && src == cgtGPU)
                 ? cgt_amd_memcpy_async((int)dest, (int)src, dest_ptr, src_ptr, nbytes, cgt_get_stream())
                 : cgt_amd_memcpy((int)dest, (int)src, dest_ptr, src_ptr, nbytes);
    cgt_check(rc == CGT_AMD_OK, "cgt_memcpy: %s", cgt_amd_last_error());
}

// ------------------------------------------------------------------ objects

static long* dup_shape(int ndim, const long* shape) {
    long* s = new long[ndim > 0 ? ndim : 1];
    for (int i = 0; i < ndim; ++i) s[i] = shape[i];
    return s;
}

cgtArray::cgtArray(int ndim, const long* shape, cgtDtype dtype, cgtDevtype devtype)
    : cgtObject(ArrayKind), ndim_(ndim), shape_(dup_shape(ndim, shape)), dtype_(dtype),
      devtype_(devtype), owns_(true), data_(NULL) {
    data_ = cgt_alloc(devtype_, nbytes());
}

cgtArray::cgtArray(int ndim, const long* shape, cgtDtype dtype, cgtDevtype devtype, void* fromdata,
                   bool copy)
    : cgtObject(ArrayKind), ndim_(ndim), shape_(dup_shape(ndim, shape)), dtype_(dtype),
      devtype_(devtype), owns_(copy), data_(fromdata) {
    cgt_assert(fromdata != NULL);
    if (copy) {
        data_ = cgt_alloc(devtype_, nbytes());
        cgt_memcpy(devtype_, cgtCPU, data_, fromdata, nbytes());
    }
}

cgtArray::~cgtArray() {
    if (owns_ && data_) cgt_free(devtype_, data_);
    delete[] shape_;
}

void cgtArray::print() {
    printf("Array{shape=(");
    for (int i = 0; i < ndim_; ++i) printf(i ? ", %ld" : "%ld", shape_[i]);
    printf("), dtype=%d, dev=%s}", (int)dtype_, devtype_ == cgtGPU ? "gpu" : "cpu");
}

cgtTuple::cgtTuple(int n) : cgtObject(TupleKind), len(n), members(new IRC<cgtObject>[n > 0 ? n : 1]) {}

cgtTuple::~cgtTuple() { delete[] members; }

void cgt_copy_array(cgtArray* to, cgtArray* from) {
    cgt_assert(to->size() == from->size() && to->dtype() == from->dtype());
    cgt_memcpy(to->devtype(), from->devtype(), to->data(), from->data(), from->nbytes());
}

void cgt_copy_tuple(cgtTuple* to, cgtTuple* from) {
    cgt_assert(to->size() == from->size());
    for (int i = 0; i < to->size(); ++i) cgt_copy_object(to->getitem(i), from->getitem(i));
}

void cgt_copy_object(cgtObject* to, cgtObject* from) {
    cgt_assert(to->kind() == from->kind());
    if (cgt_is_array(to)) cgt_copy_array(static_cast<cgtArray*>(to), static_cast<cgtArray*>(from));
    else if (cgt_is_tuple(to)) cgt_copy_tuple(static_cast<cgtTuple*>(to), static_cast<cgtTuple*>(from));
    else cgt_assert(0 && "cgt_copy_object: object of unknown kind");
}

// ------------------------------------------------------------------ interpreter

namespace {

struct MemLocation {
    long index;
    cgtDevtype devtype;
};

enum InstrKind { LoadArgumentKind = 0, AllocKind, BuildTupKind, ReturnByRefKind, ReturnByValKind, ArgTransportKind };

struct Instruction {
    InstrKind kind;
    std::vector<MemLocation> reads;
    MemLocation write;
    // LoadArgument
    int arg_index;
    // Alloc: shape comes from the int64 host scalars in `reads`.  `backing` is the largest
    // buffer this instruction has allocated so far: a later run with a shape that fits it
    // gets a view of it instead of a new allocation.
    cgtDtype dtype;
    IRC<cgtObject> backing;   // owns the memory
    IRC<cgtObject> current;   // what the last run put into the write slot: `backing` or a view of it
    long backing_bytes;
    // ReturnByRef / ReturnByVal
    void* fptr;
    void* closure;
};

// Replays an instruction list over a table of storage slots.  Outputs of
// Alloc are reused between runs while their shape is unchanged, so the op
// kernels see the same device buffers call after call.
struct Interpreter {
    std::vector<Instruction> instrs;
    std::vector<IRC<cgtObject> > storage;
    std::vector<MemLocation> outputs;
    std::vector<cgtObject*> args;

    bool fire(Instruction& in) {
        switch (in.kind) {
            case LoadArgumentKind:
                if (in.arg_index < 0 || in.arg_index >= (int)args.size()) return fail("LoadArgument: bad index");
                storage[in.write.index] = args[in.arg_index];
                return true;
            case AllocKind: {
                const int ndim = (int)in.reads.size();
                std::vector<long> shape(ndim > 0 ? ndim : 1);
                for (int i = 0; i < ndim; ++i) {
                    cgtArray* sz = static_cast<cgtArray*>(storage[in.reads[i].index].get());
                    if (!sz || sz->dtype() != cgt_i8 || sz->devtype() != cgtCPU)
                        return fail("Alloc: shape operands must be int64 host scalars");
                    shape[i] = sz->at<long>(0);
                }
                for (int i = 0; i < ndim; ++i)
                    if (shape[i] < 0) return fail("Alloc: negative extent");
                storage[in.write.index] = place(in, ndim, shape.data(), in.dtype);
                return cgtGlobalStatus == cgtStatusOK;
            }
            case ArgTransportKind: {
                // an argument on its way to the device its consumers run on: passed through
                // untouched when it is already there, else copied (cgt_copy_object, the body
                // of the reference's Transport op) into a buffer this instruction keeps
                cgtObject* src = storage[in.reads[0].index].get();
                if (!src || !cgt_is_array(src)) return fail("Transport: the argument is not an array");
                cgtArray* a = static_cast<cgtArray*>(src);
                if (a->devtype() == in.write.devtype) {
                    storage[in.write.index] = src;
                    return true;
                }
                cgtArray* dst = place(in, a->ndim(), a->shape(), a->dtype());
                if (cgtGlobalStatus != cgtStatusOK) return false;
                storage[in.write.index] = dst;
                cgt_copy_object(dst, a);
                return cgtGlobalStatus == cgtStatusOK;
            }
            case BuildTupKind: {
                cgtTuple* t = new cgtTuple((int)in.reads.size());
                for (size_t i = 0; i < in.reads.size(); ++i) t->setitem((int)i, storage[in.reads[i].index].get());
                storage[in.write.index] = t;
                return true;
            }
            case ReturnByRefKind: {
                std::vector<cgtObject*> reads(in.reads.size() + 1);
                for (size_t i = 0; i < in.reads.size(); ++i) reads[i] = storage[in.reads[i].index].get();
                cgtObject* write = storage[in.write.index].get();
                if (!write) return fail("ReturnByRef: write location is empty");
                reinterpret_cast<cgtByRefFun>(in.fptr)(in.closure, reads.data(), write);
                return cgtGlobalStatus == cgtStatusOK;
            }
            case ReturnByValKind: {
                std::vector<cgtObject*> reads(in.reads.size() + 1);
                for (size_t i = 0; i < in.reads.size(); ++i) reads[i] = storage[in.reads[i].index].get();
                storage[in.write.index] = reinterpret_cast<cgtByValFun>(in.fptr)(in.closure, reads.data());
                return cgtGlobalStatus == cgtStatusOK;
            }
        }
        return fail("unknown instruction kind");
    }

    // The array an allocating instruction hands out for this run: the one of the last run
    // while the shape is unchanged, a view of the instruction's buffer while the shape fits
    // it, a new buffer otherwise (the old one is dropped; cgt_free waits for work that
    // still uses it).
    cgtArray* place(Instruction& in, int ndim, const long* shape, cgtDtype dtype) {
        cgtArray* cur = static_cast<cgtArray*>(in.current.get());
        bool same = cur && cur->ndim() == ndim && cur->dtype() == dtype;
        for (int i = 0; same && i < ndim; ++i) same = cur->shape()[i] == shape[i];
        if (same) return cur;
        long need = cgt_itemsize(dtype);
        for (int i = 0; i < ndim; ++i) need *= shape[i];
        cgtArray* out;
        if (in.backing && need <= in.backing_bytes) {
            cgtArray* b = static_cast<cgtArray*>(in.backing.get());
            out = new cgtArray(ndim, shape, dtype, in.write.devtype, b->data(), false);
            out->set_base(b);       // whoever keeps the view keeps the buffer
        } else {
            out = new cgtArray(ndim, shape, dtype, in.write.devtype);
            in.backing = out;
            in.backing_bytes = need;
        }
        in.current = out;
        return out;
    }

    bool fail(const char* msg) {
        cgt_check(false, "interpreter: %s", msg);
        return false;
    }
};

}  // namespace

// ------------------------------------------------------------------ C API for the host language

extern "C" {

CGT_EXPORT int cgt_rt_status(void) { return (int)cgtGlobalStatus; }
CGT_EXPORT const char* cgt_rt_error(void) { return cgtGlobalErrorMsg; }
CGT_EXPORT void cgt_rt_clear_error(void) { cgtGlobalStatus = cgtStatusOK; cgtGlobalErrorMsg[0] = 0; }

// New array with owned storage (refcount 1, release with cgt_rt_release).
CGT_EXPORT void* cgt_rt_array_new(int ndim, const long* shape, int dtype, int devtype) {
    cgtArray* a = new cgtArray(ndim, shape, (cgtDtype)dtype, (cgtDevtype)devtype);
    a->Retain();
    return a;
}

// Non-owning view of memory that already lives on `devtype`.
CGT_EXPORT void* cgt_rt_array_view(int ndim, const long* shape, int dtype, int devtype, void* data) {
    cgtArray* a = new cgtArray(ndim, shape, (cgtDtype)dtype, (cgtDevtype)devtype, data, false);
    a->Retain();
    return a;
}

CGT_EXPORT void* cgt_rt_tuple_new(int len) {
    cgtTuple* t = new cgtTuple(len);
    t->Retain();
    return t;
}

CGT_EXPORT void cgt_rt_tuple_setitem(void* tup, int i, void* obj) {
    static_cast<cgtTuple*>(static_cast<cgtObject*>(tup))->setitem(i, static_cast<cgtObject*>(obj));
}

CGT_EXPORT void* cgt_rt_tuple_getitem(void* tup, int i) {
    return static_cast<cgtTuple*>(static_cast<cgtObject*>(tup))->getitem(i);
}

CGT_EXPORT int cgt_rt_tuple_len(void* tup) { return static_cast<cgtTuple*>(static_cast<cgtObject*>(tup))->size(); }
CGT_EXPORT void cgt_rt_retain(void* obj) { static_cast<cgtObject*>(obj)->Retain(); }
CGT_EXPORT void cgt_rt_release(void* obj) { if (obj) static_cast<cgtObject*>(obj)->Release(); }
CGT_EXPORT int cgt_rt_kind(void* obj) { return (int)static_cast<cgtObject*>(obj)->kind(); }

static cgtArray* as_array(void* obj) { return static_cast<cgtArray*>(static_cast<cgtObject*>(obj)); }
CGT_EXPORT int cgt_rt_array_ndim(void* a) { return as_array(a)->ndim(); }
CGT_EXPORT const long* cgt_rt_array_shape(void* a) { return as_array(a)->shape(); }
CGT_EXPORT int cgt_rt_array_dtype(void* a) { return (int)as_array(a)->dtype(); }
CGT_EXPORT int cgt_rt_array_devtype(void* a) { return (int)as_array(a)->devtype(); }
CGT_EXPORT void* cgt_rt_array_data(void* a) { return as_array(a)->data(); }
CGT_EXPORT long cgt_rt_array_nbytes(void* a) { return as_array(a)->nbytes(); }
CGT_EXPORT long cgt_rt_array_stride(void* a, int i) { return as_array(a)->stride(i); }

CGT_EXPORT int cgt_rt_copy_object(void* to, void* from) {
    cgt_copy_object(static_cast<cgtObject*>(to), static_cast<cgtObject*>(from));
    return (int)cgtGlobalStatus;
}

// Fire one compiled by-reference closure; returns the status afterwards.
CGT_EXPORT int cgt_rt_apply_byref(void* fptr, void* closure, void** reads, int n_reads, void* write) {
    std::vector<cgtObject*> r(n_reads + 1);
    for (int i = 0; i < n_reads; ++i) r[i] = static_cast<cgtObject*>(reads[i]);
    reinterpret_cast<cgtByRefFun>(fptr)(closure, r.data(), static_cast<cgtObject*>(write));
    return (int)cgtGlobalStatus;
}

// Fire one compiled by-value closure; the result comes back with refcount 1.
CGT_EXPORT void* cgt_rt_apply_byval(void* fptr, void* closure, void** reads, int n_reads) {
    std::vector<cgtObject*> r(n_reads + 1);
    for (int i = 0; i < n_reads; ++i) r[i] = static_cast<cgtObject*>(reads[i]);
    cgtObject* out = reinterpret_cast<cgtByValFun>(fptr)(closure, r.data());
    if (out) out->Retain();
    return out;
}

CGT_EXPORT void* cgt_rt_interp_new(long n_slots) {
    Interpreter* it = new Interpreter();
    it->storage.resize(n_slots);
    return it;
}

CGT_EXPORT void cgt_rt_interp_free(void* h) { delete static_cast<Interpreter*>(h); }

static void fill_locs(std::vector<MemLocation>& v, const long* idx, const int* dev, int n) {
    v.resize(n);
    for (int i = 0; i < n; ++i) { v[i].index = idx[i]; v[i].devtype = (cgtDevtype)dev[i]; }
}

static int push(Interpreter* it, Instruction& in, const long* ridx, const int* rdev, int nr, long widx, int wdev) {
    const long ns = (long)it->storage.size();
    if (widx < 0 || widx >= ns) return -1;
    for (int i = 0; i < nr; ++i) if (ridx[i] < 0 || ridx[i] >= ns) return -1;
    fill_locs(in.reads, ridx, rdev, nr);
    in.write.index = widx;
    in.write.devtype = (cgtDevtype)wdev;
    it->instrs.push_back(in);
    return (int)it->instrs.size() - 1;
}

CGT_EXPORT int cgt_rt_interp_add_load_argument(void* h, int arg_index, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = LoadArgumentKind;
    in.arg_index = arg_index;
    return push(static_cast<Interpreter*>(h), in, NULL, NULL, 0, widx, wdev);
}

CGT_EXPORT int cgt_rt_interp_add_alloc(void* h, int dtype, const long* ridx, const int* rdev, int nr, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = AllocKind;
    in.dtype = (cgtDtype)dtype;
    return push(static_cast<Interpreter*>(h), in, ridx, rdev, nr, widx, wdev);
}

CGT_EXPORT int cgt_rt_interp_add_arg_transport(void* h, long ridx, int rdev, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = ArgTransportKind;
    return push(static_cast<Interpreter*>(h), in, &ridx, &rdev, 1, widx, wdev);
}

CGT_EXPORT int cgt_rt_interp_add_build_tup(void* h, const long* ridx, const int* rdev, int nr, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = BuildTupKind;
    return push(static_cast<Interpreter*>(h), in, ridx, rdev, nr, widx, wdev);
}

CGT_EXPORT int cgt_rt_interp_add_return_byref(void* h, void* fptr, void* closure, const long* ridx, const int* rdev, int nr, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = ReturnByRefKind;
    in.fptr = fptr;
    in.closure = closure;
    return push(static_cast<Interpreter*>(h), in, ridx, rdev, nr, widx, wdev);
}

CGT_EXPORT int cgt_rt_interp_add_return_byval(void* h, void* fptr, void* closure, const long* ridx, const int* rdev, int nr, long widx, int wdev) {
    Instruction in = Instruction();
    in.kind = ReturnByValKind;
    in.fptr = fptr;
    in.closure = closure;
    return push(static_cast<Interpreter*>(h), in, ridx, rdev, nr, widx, wdev);
}

// ---- shape arithmetic: by-value closures the interpreter fires through ReturnByVal, so that
// Alloc and the ops' shape operands follow the shapes of the arguments at every run (the
// reference computes them with its Size op and integer elementwise ops, cgt/core.py:1614-1640)

struct cgt_rt_size_closure { int axis; };
struct cgt_rt_intop_closure { int op; };

static cgtArray* new_i8_scalar(long v) {
    long shape1[1] = {1};
    cgtArray* a = new cgtArray(0, shape1, cgt_i8, cgtCPU);
    a->at<long>(0) = v;
    return a;
}

// extent of axis `axis` of reads[0] as an int64 host scalar
CGT_EXPORT cgtObject* cgt_rt_op_size(void* cl, cgtObject** reads) {
    const int axis = static_cast<cgt_rt_size_closure*>(cl)->axis;
    cgtArray* a = static_cast<cgtArray*>(reads[0]);
    cgt_check(cgt_is_array(reads[0]) && axis >= 0 && axis < a->ndim(), "Size: axis %d of a %d-d array", axis, a->ndim());
    if (cgtGlobalStatus != cgtStatusOK) return new_i8_scalar(0);
    return new_i8_scalar(a->shape()[axis]);
}

// integer arithmetic on int64 host scalars: 0 add, 1 sub, 2 mul, 3 floor division,
// 4 max(0, ceil(x / y)) (the pooling size rule), 5 negate (one operand)
CGT_EXPORT cgtObject* cgt_rt_op_intop(void* cl, cgtObject** reads) {
    const int op = static_cast<cgt_rt_intop_closure*>(cl)->op;
    const long x = static_cast<cgtArray*>(reads[0])->at<long>(0);
    const long y = op == 5 ? 1 : static_cast<cgtArray*>(reads[1])->at<long>(0);
    long r = 0;
    cgt_check(!((op == 3 || op == 4) && y == 0), "integer division by zero in a shape expression");
    if (cgtGlobalStatus != cgtStatusOK) return new_i8_scalar(0);
    switch (op) {
        case 0: r = x + y; break;
        case 1: r = x - y; break;
        case 2: r = x * y; break;
        case 3: r = x / y - ((x % y != 0) && ((x < 0) != (y < 0)) ? 1 : 0); break;   // floor, like python //
        case 4: {
            long f = x / y - ((x % y != 0) && ((x < 0) != (y < 0)) ? 1 : 0);
            long c = f + (x % y != 0 ? 1 : 0);
            r = c > 0 ? c : 0;
            break;
        }
        case 5: r = -x; break;
        default: cgt_check(false, "unknown integer op %d", op);
    }
    return new_i8_scalar(r);
}

// Pre-load a constant (e.g. a shape scalar or a parameter) into a slot.
CGT_EXPORT int cgt_rt_interp_set_slot(void* h, long idx, void* obj) {
    Interpreter* it = static_cast<Interpreter*>(h);
    if (idx < 0 || idx >= (long)it->storage.size()) return -1;
    it->storage[idx] = static_cast<cgtObject*>(obj);
    return 0;
}

// Borrowed pointer to what a slot holds after a run (NULL if empty).
CGT_EXPORT void* cgt_rt_interp_get_slot(void* h, long idx) {
    Interpreter* it = static_cast<Interpreter*>(h);
    if (idx < 0 || idx >= (long)it->storage.size()) return NULL;
    return it->storage[idx].get();
}

// Run every instruction in order.  Returns 0, or 1 + the index of the
// instruction that failed (message in cgt_rt_error()).
CGT_EXPORT int cgt_rt_interp_run(void* h, void** args, int n_args) {
    Interpreter* it = static_cast<Interpreter*>(h);
    it->args.resize(n_args);
    for (int i = 0; i < n_args; ++i) it->args[i] = static_cast<cgtObject*>(args[i]);
    for (size_t i = 0; i < it->instrs.size(); ++i)
        if (!it->fire(it->instrs[i])) return 1 + (int)i;
    it->args.clear();
    return 0;
}

}  // extern "C"
