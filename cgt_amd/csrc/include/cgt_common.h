// Runtime object model seen by compiled op closures:
//     void call_X(closure*, cgtArray** reads, cgtArray* | cgtTuple* write)
// Source-compatible with the names CGT op bodies use (cgtArray::shape(),
// data(), stride(), at<T>(), cgtTuple::getitem(), CGT_EXPORT_C, cgt_assert,
// cgt_check, cgt_alloc/free/memcpy; reference include/cgt_common.h:14-227),
// written for a HIP device behind devtype cgtGPU: device memory comes from
// libcgt_amd (cgt_amd_alloc), strides are 64-bit, and failures are recorded
// in a status the host reads back instead of being printed.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdio>
#include <cstdlib>

#define CGT_EXPORT __attribute__((visibility("default")))
#define CGT_EXPORT_C extern "C" __attribute__((visibility("default")))
#define CGT_NORETURN __attribute__((noreturn))

// ------------------------------------------------------------------ scalars

// numpy type numbers (np.dtype(...).num), as the host side hands them over
typedef enum cgtDtype {
    cgt_i1 = 1, cgt_i2 = 3, cgt_i4 = 5, cgt_i8 = 7,
    cgt_f2 = 23, cgt_f4 = 11, cgt_f8 = 12, cgt_f16 = 13,
    cgt_c8 = 14, cgt_c16 = 15, cgt_c32 = 16, cgt_O = 17
} cgtDtype;

static inline int cgt_itemsize(cgtDtype d) {
    switch (d) {
        case cgt_i1: return 1;
        case cgt_i2: case cgt_f2: return 2;
        case cgt_i4: case cgt_f4: return 4;
        case cgt_i8: case cgt_f8: case cgt_c8: case cgt_O: return 8;
        case cgt_f16: case cgt_c16: return 16;
        case cgt_c32: return 32;
    }
    return -1;
}

typedef enum cgtDevtype { cgtCPU = 0, cgtGPU = 1 } cgtDevtype;

// ------------------------------------------------------------------ errors

typedef enum { cgtStatusOK = 0, cgtStatusErr } cgtStatus;
extern "C" CGT_EXPORT cgtStatus cgtGlobalStatus;
extern "C" CGT_EXPORT char cgtGlobalErrorMsg[1000];

static inline void clear_error() { cgtGlobalStatus = cgtStatusOK; }

// Records the failure; the host checks cgtGlobalStatus after the closure returns.
#define cgt_check(cond, ...)                                                   \
    do {                                                                       \
        if (!(cond)) {                                                         \
            snprintf(cgtGlobalErrorMsg, sizeof(cgtGlobalErrorMsg), __VA_ARGS__); \
            cgtGlobalStatus = cgtStatusErr;                                    \
        }                                                                      \
    } while (0)

#define cgt_assert(cond)                                                          \
    do {                                                                          \
        if (!(cond)) {                                                            \
            fprintf(stderr, "Assertion failed: %s (%s:%d)\n", #cond, __FILE__, __LINE__); \
            fflush(stderr);                                                       \
            abort();                                                              \
        }                                                                         \
    } while (0)

// ------------------------------------------------------------------ memory

CGT_EXPORT void* cgt_alloc(cgtDevtype devtype, long nbytes);
CGT_EXPORT void cgt_free(cgtDevtype devtype, void* ptr);
CGT_EXPORT void cgt_memcpy(cgtDevtype dest, cgtDevtype src, void* dest_ptr, void* src_ptr, long nbytes);

// The HIP stream op closures launch on (NULL = default stream).
extern "C" CGT_EXPORT void* cgt_get_stream(void);
extern "C" CGT_EXPORT void cgt_set_stream(void* stream);

// ------------------------------------------------------------------ refcounting

// Intrusive pointer: the pointee carries the count (Retain / Release).
template <typename T>
class IRC {
public:
    IRC() : p_(NULL) {}
    IRC(T* p) : p_(p) { if (p_) p_->Retain(); }
    IRC(const IRC& o) : p_(o.p_) { if (p_) p_->Retain(); }
    template <typename U>
    IRC(const IRC<U>& o) : p_(o.get()) { if (p_) p_->Retain(); }
    ~IRC() { if (p_) p_->Release(); }
    IRC& operator=(IRC o) { swap(o); return *this; }
    void swap(IRC& o) { T* t = p_; p_ = o.p_; o.p_ = t; }
    void reset() { IRC().swap(*this); }
    T* get() const { return p_; }
    T& operator*() const { return *p_; }
    T* operator->() const { return p_; }
    operator bool() const { return p_ != NULL; }
private:
    T* p_;
};

// ------------------------------------------------------------------ objects

class CGT_EXPORT cgtObject {
public:
    enum ObjectKind { UndefKind = 0, ArrayKind, TupleKind };
    explicit cgtObject(ObjectKind kind = UndefKind) : kind_(kind), refs_(0) {}
    virtual ~cgtObject() {}
    ObjectKind kind() const { return kind_; }
    void Retain() const { refs_.fetch_add(1, std::memory_order_relaxed); }
    void Release() const {
        if (refs_.fetch_sub(1, std::memory_order_acq_rel) == 1) delete this;
    }
    unsigned refcount() const { return refs_.load(); }
private:
    ObjectKind kind_;
    mutable std::atomic<unsigned> refs_;
};

// Contiguous row-major n-d array on the host or in HBM.
class CGT_EXPORT cgtArray : public cgtObject {
public:
    // fresh, owned storage
    cgtArray(int ndim, const long* shape, cgtDtype dtype, cgtDevtype devtype);
    // copy = true: owned copy of host data `fromdata`; copy = false: view of
    // `fromdata`, which already lives on `devtype`
    cgtArray(int ndim, const long* shape, cgtDtype dtype, cgtDevtype devtype, void* fromdata, bool copy);
    ~cgtArray();

    int ndim() const { return ndim_; }
    const long* shape() const { return shape_; }
    long size() const {
        long n = 1;
        for (int i = 0; i < ndim_; ++i) n *= shape_[i];
        return n;
    }
    long nbytes() const { return size() * cgt_itemsize(dtype_); }
    // elements between consecutive indices of axis i
    long stride(int i) const {
        if (ndim_ == 0) return 0;
        long s = 1;
        for (int j = ndim_ - 1; j > i; --j) s *= shape_[j];
        return s;
    }
    cgtDtype dtype() const { return dtype_; }
    cgtDevtype devtype() const { return devtype_; }
    bool ownsdata() const { return owns_; }
    void* data() { return data_; }

    // host-side element access (valid for cgtCPU arrays only)
    template <typename T> T& at() { return static_cast<T*>(data_)[0]; }
    template <typename T> T& at(long i) { return static_cast<T*>(data_)[i]; }
    template <typename T> T& at(long i, long j) { return static_cast<T*>(data_)[i * shape_[1] + j]; }
    template <typename T> T& at(long i, long j, long k) {
        return static_cast<T*>(data_)[(i * shape_[1] + j) * shape_[2] + k];
    }
    template <typename T> T& at(long i, long j, long k, long l) {
        return static_cast<T*>(data_)[((i * shape_[1] + j) * shape_[2] + k) * shape_[3] + l];
    }
    void print();

    // A view (ownsdata() false) may name the object whose storage it shows: that object then
    // lives at least as long as the view.  The interpreter's views of its instruction buffers
    // and Reshape's results do, so an output a caller keeps stays valid when a later call
    // makes the interpreter drop the buffer for a larger one.
    void set_base(cgtObject* base) { base_ = base; }
    cgtObject* base() const { return base_.get(); }

private:
    int ndim_;
    long* shape_;
    cgtDtype dtype_;
    cgtDevtype devtype_;
    bool owns_;
    void* data_;
    IRC<cgtObject> base_;       // last member: the offsets of the fields above are those of earlier builds
};

class CGT_EXPORT cgtTuple : public cgtObject {
public:
    explicit cgtTuple(int len);
    ~cgtTuple();
    void setitem(int i, cgtObject* o) { members[i] = o; }
    cgtObject* getitem(int i) { return members[i].get(); }
    int size() { return len; }
    int len;
    IRC<cgtObject>* members;
};

static inline bool cgt_is_array(cgtObject* o) { return o->kind() == cgtObject::ArrayKind; }
static inline bool cgt_is_tuple(cgtObject* o) { return o->kind() == cgtObject::TupleKind; }

// Copy `from` into `to`, crossing host <-> device as their devtypes require.
CGT_EXPORT void cgt_copy_object(cgtObject* to, cgtObject* from);
CGT_EXPORT void cgt_copy_array(cgtArray* to, cgtArray* from);
CGT_EXPORT void cgt_copy_tuple(cgtTuple* to, cgtTuple* from);

// Compiled op entry points.
typedef void (*cgtByRefFun)(void* closure, cgtObject** reads, cgtObject* write);
typedef cgtObject* (*cgtByValFun)(void* closure, cgtObject** reads);
