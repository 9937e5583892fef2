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
    int rc = cgt_amd_memcpy((int)dest, (int)src, dest_ptr, src_ptr, nbytes);
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

enum InstrKind { LoadArgumentKind = 0, AllocKind, BuildTupKind, ReturnByRefKind, ReturnByValKind };

struct Instruction {
    InstrKind kind;
    std::vector<MemLocation> reads;
    MemLocation write;
    // LoadArgument
    int arg_index;
    // Alloc: shape comes from the int64 host scalars in `reads`
    cgtDtype dtype;
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
                cgtArray* cur = static_cast<cgtArray*>(storage[in.write.index].get());
                bool same = cur && cur->kind() == cgtObject::ArrayKind && cur->ndim() == ndim &&
                            cur->dtype() == in.dtype && cur->devtype() == in.write.devtype;
                for (int i = 0; same && i < ndim; ++i) same = cur->shape()[i] == shape[i];
                if (!same) storage[in.write.index] = new cgtArray(ndim, shape.data(), in.dtype, in.write.devtype);
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
