// Python extension module dpnp_amd._dpx_ext: the binding between the Python array objects and the C ABI.
//
// Role of the reference's pybind11 layer (PYBIND11_MODULE(_tensor_elementwise_impl, m),
// libtensor/source/tensor_elementwise.cpp:42; the usm_ndarray accessors of
// dpnp/include/dpnp4pybind11.hpp:402-447; py_unary_ufunc / py_binary_ufunc,
// libtensor/source/elementwise_functions/elementwise_functions.hpp:77-251; py_reduction_over_axis,
// libtensor/source/reductions/reduction_over_axis.hpp:174-501): the functions take array objects, read
// shape / strides / dtype / flags / pointer from them in C++, fill dpx_array_view descriptors, call dpx_*,
// and turn a status code into the exception class the reference raises.
//
// Two kinds of functions:
//  * make_unary / make_binary / make_reduction / make_search / where / copy: the boundary functions under the
//    reference's names, _X(src..., dst, sycl_queue, depends) -> (event, event);
//  * unary_call / binary_call / reduce_call: the whole of a NumPy-style call `f(x[, y], out=out)` or
//    `sum(x, axis, out=out)` for the plain case (arrays whose dtype the kernel takes as it is, no casting,
//    no overlap): what the Python layer's checks come to for such a call, done on the descriptors.  They
//    return NotImplemented for anything else and the Python layer's general path then runs (and raises
//    what there is to raise).
//
// The descriptor of an array object is built once per object by its own `_as_view()` (a ctypes structure
// kept in the object's __dict__); this module reads that structure's memory through the buffer protocol.
#include <pybind11/pybind11.h>
#include <cstring>
#include <string>
#include "../../include/dpnp_amd.h"

namespace py = pybind11;

namespace {

PyObject *s_cview, *s_as_view, *s_writable, *s_array_obj; // interned attribute names
PyTypeObject *g_usm_type = nullptr, *g_dpnp_type = nullptr;
PyObject *g_stream_fn = nullptr; // callable(device_index) -> hipStream_t as int
bool g_stream_fixed = false;     // the callable always gives the same stream (the library's own): asked once
void *g_stream = nullptr;        // that stream, once known
PyObject *g_events = nullptr;    // the (event, event) pair of the default queue
PyObject *g_events_fn = nullptr; // callable(queue) -> (event, event)
PyObject *g_alloc = nullptr;     // callable(shape tuple, dtype id) -> freshly allocated C-contiguous usm_ndarray
PyObject *g_wrap = nullptr;      // callable(usm_ndarray) -> dpnp_array

// result dtype of `op(dt)` / `op(dt, dt)` when the kernel takes the input dtype as it is and the Python
// layer's type search accepts it: -2 not looked up yet, -1 no, else the dtype id.  Filled by the Python
// layer, which owns the type search.
int8_t g_unary_res[128][DPX_NUM_DTYPES], g_binary_res[128][DPX_NUM_DTYPES];
// default result dtype of reduction / search `op` for an input dtype (dtype=None)
int8_t g_reduce_res[64][DPX_NUM_DTYPES], g_search_res[16][DPX_NUM_DTYPES];

[[noreturn]] void raise_status(int status)
{
    const char *msg = dpx_last_error();
    PyObject *exc = (status == DPX_ERR_NOT_IMPLEMENTED || status == DPX_ERR_HIP) ? PyExc_RuntimeError : PyExc_ValueError;
    PyErr_SetString(exc, msg ? msg : "dpnp_amd: unknown failure");
    throw py::error_already_set();
}

inline PyObject *dict_get(PyObject *obj, PyObject *name)
{
    PyObject **dp = _PyObject_GetDictPtr(obj);
    return (dp && *dp) ? PyDict_GetItemWithError(*dp, name) : nullptr; // borrowed
}

// usm_ndarray of a dpnp_array, or the usm_ndarray itself; null for anything else (exact types only)
inline PyObject *usm_of(PyObject *o)
{
    if (Py_TYPE(o) == g_usm_type) return o;
    if (Py_TYPE(o) == g_dpnp_type) {
        PyObject *u = dict_get(o, s_array_obj);
        if (u && Py_TYPE(u) == g_usm_type) return u;
    }
    return nullptr;
}

// The descriptor kept with a usm_ndarray (built by its _as_view() on first use), writable bit refreshed.
dpx_array_view *view_of(PyObject *u)
{
    PyObject *cv = dict_get(u, s_cview);
    if (!cv) {
        PyObject *r = PyObject_CallMethodNoArgs(u, s_as_view); // builds and keeps it
        if (!r) throw py::error_already_set();
        Py_DECREF(r);
        cv = dict_get(u, s_cview);
        if (!cv) throw py::type_error("array object without a descriptor");
    }
    Py_buffer b;
    if (PyObject_GetBuffer(cv, &b, PyBUF_SIMPLE) < 0) throw py::error_already_set();
    dpx_array_view *v = (dpx_array_view *)b.buf;
    const bool ok = (size_t)b.len >= sizeof(dpx_array_view);
    PyBuffer_Release(&b); // the structure lives as long as the array object does
    if (!ok) throw py::type_error("array descriptor of unexpected size");
    PyObject *w = dict_get(u, s_writable);
    if (w) v->flags = (v->flags & ~DPX_WRITABLE) | (PyObject_IsTrue(w) ? DPX_WRITABLE : 0);
    return v;
}

dpx_array_view *view_arg(py::handle h, const char *what)
{
    PyObject *u = usm_of(h.ptr());
    if (!u) {
        // subclasses and look-alikes: anything with _as_view()
        if (PyObject_HasAttr(h.ptr(), s_as_view)) return view_of(h.ptr());
        throw py::type_error(std::string(what) + ": expected a usm_ndarray, got " + Py_TYPE(h.ptr())->tp_name);
    }
    return view_of(u);
}

void *stream_of(py::handle queue)
{
    if (!queue.is_none()) return (void *)py::cast<uintptr_t>(queue.attr("stream_ptr"));
    if (g_stream) return g_stream;
    PyObject *zero = PyLong_FromLong(0);
    PyObject *r = PyObject_CallOneArg(g_stream_fn, zero);
    Py_DECREF(zero);
    if (!r) throw py::error_already_set();
    void *s = PyLong_AsVoidPtr(r);
    Py_DECREF(r);
    if (!s && PyErr_Occurred()) throw py::error_already_set();
    if (g_stream_fixed) g_stream = s; // the library's own stream: one per process, created at first use
    return s;
}

py::object events_of(py::handle queue)
{
    if (queue.is_none()) return py::reinterpret_borrow<py::object>(g_events);
    return py::reinterpret_steal<py::object>(PyObject_CallOneArg(g_events_fn, queue.ptr()));
}

inline int64_t itemsize(int dt) { return dpx_dtype_itemsize(dt); }
inline int64_t view_elems(const dpx_array_view *v)
{
    int64_t n = 1;
    for (int d = 0; d < v->nd; ++d) n *= v->shape[d];
    return n;
}
inline bool same_shape(const dpx_array_view *a, const dpx_array_view *b)
{
    if (a->nd != b->nd) return false;
    for (int d = 0; d < a->nd; ++d)
        if (a->shape[d] != b->shape[d]) return false;
    return true;
}
// two C-contiguous arrays share at least one byte
inline bool spans_meet(const dpx_array_view *a, const dpx_array_view *b)
{
    const char *a0 = (const char *)a->data, *a1 = a0 + view_elems(a) * itemsize(a->dtype);
    const char *b0 = (const char *)b->data, *b1 = b0 + view_elems(b) * itemsize(b->dtype);
    return a0 < b1 && b0 < a1;
}
// `o` can be written directly by a kernel that produces a C-contiguous array of v's shape and dtype `dt`
inline bool plain_out(const dpx_array_view *o, const dpx_array_view *like, int dt)
{
    return o->dtype == dt && (o->flags & DPX_WRITABLE) && (o->flags & DPX_C_CONTIGUOUS) && same_shape(o, like);
}

py::object not_implemented() { return py::reinterpret_borrow<py::object>(Py_NotImplemented); }

// A fresh C-contiguous array of `shape` and dtype id `dt`, of the class of `like` (dpnp_array or usm_ndarray).
// Returns the object to hand back and sets *view to its descriptor.
py::object fresh_result(PyObject *like, const int64_t *shape, int nd, int dt, dpx_array_view **view)
{
    py::tuple shp(nd);
    for (int d = 0; d < nd; ++d) shp[d] = py::int_(shape[d]);
    py::object u = py::reinterpret_steal<py::object>(PyObject_CallFunctionObjArgs(g_alloc, shp.ptr(), py::int_(dt).ptr(), nullptr));
    if (!u) throw py::error_already_set();
    *view = view_of(u.ptr());
    if (Py_TYPE(like) == g_dpnp_type) {
        py::object w = py::reinterpret_steal<py::object>(PyObject_CallOneArg(g_wrap, u.ptr()));
        if (!w) throw py::error_already_set();
        return w;
    }
    return u;
}

// ---------------------------------------------------------------------------------------------------------
// Broadcast descriptors of `n` operands against each other: extent 1 -> stride 0.  False when the shapes do
// not broadcast (the general path words the error) or the result is empty.
bool broadcast_views(const dpx_array_view *const *in, int n, dpx_array_view *b, int64_t *shape, int *nd_out, bool *plain)
{
    int nd = 0;
    for (int i = 0; i < n; ++i) nd = in[i]->nd > nd ? in[i]->nd : nd;
    for (int d = 0; d < nd; ++d) shape[d] = 1;
    for (int i = 0; i < n; ++i)
        for (int d = 0; d < in[i]->nd; ++d) {
            const int k = nd - in[i]->nd + d;
            if (in[i]->shape[d] == 1) continue;
            if (shape[k] == 1) shape[k] = in[i]->shape[d];
            else if (shape[k] != in[i]->shape[d]) return false;
        }
    int64_t total = 1;
    for (int d = 0; d < nd; ++d) total *= shape[d];
    if (total == 0) return false;
    *plain = true; // nothing broadcast, all C-contiguous
    for (int i = 0; i < n; ++i) {
        b[i] = *in[i];
        b[i].nd = nd;
        bool same = in[i]->nd == nd;
        for (int d = 0; d < nd; ++d) {
            const int k = d - (nd - in[i]->nd);
            const int64_t ext = k >= 0 ? in[i]->shape[k] : 1;
            b[i].shape[d] = shape[d];
            b[i].strides[d] = (k >= 0 && ext == shape[d]) ? in[i]->strides[k] : 0;
            same = same && ext == shape[d];
        }
        if (!same) b[i].flags &= ~(DPX_C_CONTIGUOUS | DPX_F_CONTIGUOUS);
        b[i].flags &= ~DPX_WRITABLE;
        *plain = *plain && same && (in[i]->flags & DPX_C_CONTIGUOUS);
    }
    *nd_out = nd;
    return true;
}

// `out` as the destination of a kernel that produces `shape` of dtype `dt`: right type and shape, writable, and
// sharing no memory with an input (the in-place and temporary cases belong to the general path)
dpx_array_view *checked_out(py::handle out, PyObject *like, const int64_t *shape, int nd, int dt,
                            const dpx_array_view *const *in, int n)
{
    PyObject *uo = usm_of(out.ptr());
    if (!uo || Py_TYPE(out.ptr()) != Py_TYPE(like)) return nullptr;
    dpx_array_view *vo = view_of(uo);
    if (vo->dtype != dt || !(vo->flags & DPX_WRITABLE) || vo->nd != nd) return nullptr;
    for (int d = 0; d < nd; ++d)
        if (vo->shape[d] != shape[d]) return nullptr;
    for (int i = 0; i < n; ++i)
        if (dpx_array_overlap(in[i], vo)) return nullptr;
    return vo;
}

// f(x, out=out) for an array whose dtype the kernel takes as it is.  A fresh result is made here only for a
// C-contiguous x (its layout is then C); with `out` any layout of x goes.
py::object unary_call(int op, py::handle x, py::handle out)
{
    PyObject *ux = usm_of(x.ptr());
    if (!ux || op < 0 || op >= 128) return not_implemented();
    dpx_array_view *vx = view_of(ux);
    const int rdt = g_unary_res[op][vx->dtype];
    if (rdt < 0) return not_implemented();
    dpx_array_view *vo;
    py::object res;
    if (out.is_none()) {
        if (!(vx->flags & DPX_C_CONTIGUOUS)) return not_implemented();
        res = fresh_result(x.ptr(), vx->shape, vx->nd, rdt, &vo);
    }
    else {
        if (view_elems(vx) == 0) return not_implemented();
        const dpx_array_view *in[1] = {vx};
        vo = checked_out(out, x.ptr(), vx->shape, vx->nd, rdt, in, 1);
        if (!vo) return not_implemented();
        res = py::reinterpret_borrow<py::object>(out);
    }
    if (int rc = dpx_unary(op, vx, vo, stream_of(py::none()))) raise_status(rc);
    return res;
}

// f(x1, x2, out=out) for two arrays of one dtype that the kernel takes as it is.  A fresh result is made here
// only for two C-contiguous arrays of one shape; with `out` the operands may have any layout and broadcast.
py::object binary_call(int op, py::handle x1, py::handle x2, py::handle out)
{
    PyObject *u1 = usm_of(x1.ptr()), *u2 = usm_of(x2.ptr());
    if (!u1 || !u2 || Py_TYPE(x1.ptr()) != Py_TYPE(x2.ptr()) || op < 0 || op >= 128) return not_implemented();
    dpx_array_view *v1 = view_of(u1), *v2 = view_of(u2);
    if (v1->dtype != v2->dtype) return not_implemented();
    const int rdt = g_binary_res[op][v1->dtype];
    if (rdt < 0) return not_implemented();
    dpx_array_view *vo;
    py::object res;
    if (out.is_none()) {
        if (!(v1->flags & v2->flags & DPX_C_CONTIGUOUS) || !same_shape(v1, v2)) return not_implemented();
        res = fresh_result(x1.ptr(), v1->shape, v1->nd, rdt, &vo);
        if (int rc = dpx_binary(op, v1, v2, vo, stream_of(py::none()))) raise_status(rc);
        return res;
    }
    if (out.ptr() == x1.ptr()) return not_implemented(); // x1 op= x2: the in-place kernels, general path
    const dpx_array_view *in[2] = {v1, v2};
    dpx_array_view b[2];
    int64_t shape[DPX_MAX_ND];
    int nd;
    bool plain;
    if (!broadcast_views(in, 2, b, shape, &nd, &plain)) return not_implemented();
    vo = checked_out(out, x1.ptr(), shape, nd, rdt, in, 2);
    if (!vo) return not_implemented();
    if (int rc = dpx_binary(op, plain ? v1 : &b[0], plain ? v2 : &b[1], vo, stream_of(py::none()))) raise_status(rc);
    return py::reinterpret_borrow<py::object>(out);
}

// sum(x, axis=axis, out=out) and its siblings with dtype=None, keepdims=False: `axis` None, an int or a
// tuple of ints.  The reduced axes are moved last on the descriptor (a permutation of shape and strides,
// nothing is copied), as dpnp/tensor/_reduction.py:59-76 does with permute_dims.
py::object reduce_call(int op, bool search, py::handle x, py::handle axis, py::handle out)
{
    PyObject *ux = usm_of(x.ptr());
    if (!ux || op < 0 || op >= (search ? 16 : 64)) return not_implemented();
    dpx_array_view *vx = view_of(ux);
    const int nd = vx->nd;
    const int rdt = search ? g_search_res[op][vx->dtype] : g_reduce_res[op][vx->dtype];
    if (rdt < 0) return not_implemented();
    bool reduced[DPX_MAX_ND] = {false};
    int red_nd = 0;
    auto mark = [&](py::handle a) -> bool {
        if (!PyLong_CheckExact(a.ptr())) return false;
        long ax = PyLong_AsLong(a.ptr());
        if (ax == -1 && PyErr_Occurred()) {
            PyErr_Clear();
            return false;
        }
        if (ax < -nd || ax >= nd) return false; // the general path raises
        if (ax < 0) ax += nd;
        if (reduced[ax]) return false;
        reduced[ax] = true;
        ++red_nd;
        return true;
    };
    if (axis.is_none()) {
        for (int d = 0; d < nd; ++d) reduced[d] = true;
        red_nd = nd;
    }
    else if (PyTuple_CheckExact(axis.ptr())) {
        if (search) return not_implemented(); // a search takes one axis
        for (py::handle a : py::reinterpret_borrow<py::tuple>(axis))
            if (!mark(a)) return not_implemented();
    }
    else if (!mark(axis)) return not_implemented();
    if (red_nd == 0) return not_implemented();
    dpx_array_view src = *vx;
    int64_t res_shape[DPX_MAX_ND];
    int k = 0;
    for (int d = 0; d < nd; ++d)
        if (!reduced[d]) {
            src.shape[k] = vx->shape[d];
            src.strides[k] = vx->strides[d];
            res_shape[k] = vx->shape[d];
            ++k;
        }
    const int res_nd = k;
    for (int d = 0; d < nd; ++d)
        if (reduced[d]) {
            if (vx->shape[d] == 0) return not_implemented(); // empty reductions: identities and errors are the general path's
            src.shape[k] = vx->shape[d];
            src.strides[k] = vx->strides[d];
            ++k;
        }
    for (int d = 0; d < res_nd; ++d)
        if (res_shape[d] == 0) return not_implemented();
    // contiguity flags of the permuted descriptor: kept only when nothing moved
    bool moved = false;
    for (int d = 0; d < nd && !moved; ++d) moved = src.strides[d] != vx->strides[d] || src.shape[d] != vx->shape[d];
    if (moved) src.flags &= ~(DPX_C_CONTIGUOUS | DPX_F_CONTIGUOUS);
    dpx_array_view *vo;
    py::object res;
    if (out.is_none()) res = fresh_result(x.ptr(), res_shape, res_nd, rdt, &vo);
    else {
        PyObject *uo = usm_of(out.ptr());
        if (!uo || Py_TYPE(out.ptr()) != Py_TYPE(x.ptr())) return not_implemented();
        vo = view_of(uo);
        if (vo->dtype != rdt || !(vo->flags & DPX_WRITABLE) || vo->nd != res_nd) return not_implemented();
        for (int d = 0; d < res_nd; ++d)
            if (vo->shape[d] != res_shape[d]) return not_implemented();
        if (dpx_array_overlap(vx, vo)) return not_implemented(); // computed into a temporary by the general path
        res = py::reinterpret_borrow<py::object>(out);
    }
    void *s = stream_of(py::none());
    const int rc = search ? dpx_argreduce(op, &src, red_nd, vo, s) : dpx_reduce(op, &src, red_nd, vo, nullptr, s);
    if (rc) {
        if (rc == DPX_ERR_NOT_IMPLEMENTED && out.is_none()) return not_implemented(); // e.g. no kernel for the pair: cast path
        raise_status(rc);
    }
    return res;
}

// where(condition, x1, x2, out=out) for arrays whose branches share a dtype: the three operands are broadcast
// on their descriptors (extent 1 -> stride 0).  A fresh result is only made here when nothing is broadcast and
// all three are C-contiguous (its layout is then C whatever the order rule); other layouts are the general path's.
py::object where_call(py::handle cond, py::handle x1, py::handle x2, py::handle out)
{
    PyObject *uc = usm_of(cond.ptr()), *u1 = usm_of(x1.ptr()), *u2 = usm_of(x2.ptr());
    if (!uc || !u1 || !u2 || Py_TYPE(x1.ptr()) != Py_TYPE(cond.ptr()) || Py_TYPE(x2.ptr()) != Py_TYPE(cond.ptr()))
        return not_implemented();
    const dpx_array_view *in[3] = {view_of(uc), view_of(u1), view_of(u2)};
    if (in[1]->dtype != in[2]->dtype) return not_implemented();
    dpx_array_view b[3];
    int64_t shape[DPX_MAX_ND];
    int nd;
    bool plain;
    if (!broadcast_views(in, 3, b, shape, &nd, &plain)) return not_implemented();
    dpx_array_view *vo;
    py::object res;
    if (out.is_none()) {
        if (!plain) return not_implemented();
        res = fresh_result(cond.ptr(), shape, nd, in[1]->dtype, &vo);
    }
    else {
        vo = checked_out(out, cond.ptr(), shape, nd, in[1]->dtype, in, 3);
        if (!vo) return not_implemented();
        res = py::reinterpret_borrow<py::object>(out);
    }
    if (int rc = dpx_where(&b[0], &b[1], &b[2], vo, stream_of(py::none()))) raise_status(rc);
    return res;
}

// ---------------------------------------------------------------------------------------------------------
py::cpp_function make_unary(int op, const std::string &name)
{
    return py::cpp_function(
        [op](py::handle src, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vs = view_arg(src, "src"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_unary(op, vs, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::name(name.c_str()), py::arg("src"), py::arg("dst"), py::arg("sycl_queue") = py::none(),
        py::arg("depends") = py::tuple());
}
py::cpp_function make_binary(int op, const std::string &name)
{
    return py::cpp_function(
        [op](py::handle src1, py::handle src2, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *v1 = view_arg(src1, "src1"), *v2 = view_arg(src2, "src2"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_binary(op, v1, v2, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::name(name.c_str()), py::arg("src1"), py::arg("src2"), py::arg("dst"), py::arg("sycl_queue") = py::none(),
        py::arg("depends") = py::tuple());
}
py::cpp_function make_binary_inplace(int op, const std::string &name)
{
    return py::cpp_function(
        [op](py::handle lhs, py::handle rhs, py::handle sycl_queue, py::handle) {
            dpx_array_view *vl = view_arg(lhs, "lhs"), *vr = view_arg(rhs, "rhs");
            if (int rc = dpx_binary_inplace(op, vl, vr, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::name(name.c_str()), py::arg("lhs"), py::arg("rhs"), py::arg("sycl_queue") = py::none(),
        py::arg("depends") = py::tuple());
}
py::cpp_function make_reduction(int op, const std::string &name)
{
    return py::cpp_function(
        [op](py::handle src, int trailing, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vs = view_arg(src, "src"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_reduce(op, vs, trailing, vd, nullptr, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::name(name.c_str()), py::arg("src"), py::arg("trailing_dims_to_reduce"), py::arg("dst"),
        py::arg("sycl_queue") = py::none(), py::arg("depends") = py::tuple());
}
py::cpp_function make_search(int op, const std::string &name)
{
    return py::cpp_function(
        [op](py::handle src, int trailing, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vs = view_arg(src, "src"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_argreduce(op, vs, trailing, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::name(name.c_str()), py::arg("src"), py::arg("trailing_dims_to_reduce"), py::arg("dst"),
        py::arg("sycl_queue") = py::none(), py::arg("depends") = py::tuple());
}

void set_table(int8_t (*tab)[DPX_NUM_DTYPES], int rows, int op, int dt, int res)
{
    if (op < 0 || op >= rows || dt < 0 || dt >= DPX_NUM_DTYPES || res < -2 || res >= DPX_NUM_DTYPES)
        throw py::value_error("type table index out of range");
    tab[op][dt] = (int8_t)res;
}

} // namespace

PYBIND11_MODULE(_dpx_ext, m)
{
    m.doc() = "binding between dpnp_amd's array objects and the C ABI of libdpnp_amd.so";
    s_cview = PyUnicode_InternFromString("_cview");
    s_as_view = PyUnicode_InternFromString("_as_view");
    s_writable = PyUnicode_InternFromString("_writable");
    s_array_obj = PyUnicode_InternFromString("_array_obj");
    std::memset(g_unary_res, -2, sizeof g_unary_res);
    std::memset(g_binary_res, -2, sizeof g_binary_res);
    std::memset(g_reduce_res, -2, sizeof g_reduce_res);
    std::memset(g_search_res, -2, sizeof g_search_res);

    m.def("init",
          [](py::object usm_type, py::object stream_fn, bool stream_fixed, py::object events_fn, py::object alloc) {
              g_usm_type = (PyTypeObject *)usm_type.release().ptr();
              g_stream_fn = stream_fn.release().ptr();
              g_stream_fixed = stream_fixed;
              g_stream = nullptr;
              g_events = events_fn(py::none()).release().ptr();
              g_events_fn = events_fn.release().ptr();
              g_alloc = alloc.release().ptr();
          },
          "init(usm_ndarray type, stream(device index) -> hipStream_t as int, whether that is always the same "
          "stream, events(queue) -> (event, event), alloc(shape, dtype id) -> usm_ndarray)");
    m.def("set_array_class", [](py::object dpnp_type, py::object wrap) {
        g_dpnp_type = (PyTypeObject *)dpnp_type.release().ptr();
        g_wrap = wrap.release().ptr();
    });
    m.def("make_unary", &make_unary);
    m.def("make_binary", &make_binary);
    m.def("make_binary_inplace", &make_binary_inplace);
    m.def("make_reduction", &make_reduction);
    m.def("make_search", &make_search);
    m.def("set_unary_type", [](int op, int dt, int res) { set_table(g_unary_res, 128, op, dt, res); });
    m.def("set_binary_type", [](int op, int dt, int res) { set_table(g_binary_res, 128, op, dt, res); });
    m.def("set_reduce_type", [](int op, int dt, int res) { set_table(g_reduce_res, 64, op, dt, res); });
    m.def("set_search_type", [](int op, int dt, int res) { set_table(g_search_res, 16, op, dt, res); });
    m.def("unary_type", [](int op, int dt) { return (int)g_unary_res[op & 127][dt % DPX_NUM_DTYPES]; });
    m.def("binary_type", [](int op, int dt) { return (int)g_binary_res[op & 127][dt % DPX_NUM_DTYPES]; });
    m.def("unary_call", &unary_call, py::arg("op"), py::arg("x"), py::arg("out") = py::none());
    m.def("binary_call", &binary_call, py::arg("op"), py::arg("x1"), py::arg("x2"), py::arg("out") = py::none());
    m.def("reduce_call", [](int op, py::handle x, py::handle axis, py::handle out) { return reduce_call(op, false, x, axis, out); },
          py::arg("op"), py::arg("x"), py::arg("axis") = py::none(), py::arg("out") = py::none());
    m.def("search_call", [](int op, py::handle x, py::handle axis, py::handle out) { return reduce_call(op, true, x, axis, out); },
          py::arg("op"), py::arg("x"), py::arg("axis") = py::none(), py::arg("out") = py::none());
    m.def("where_call", &where_call, py::arg("condition"), py::arg("x1"), py::arg("x2"), py::arg("out") = py::none());
    m.def(
        "_where",
        [](py::handle condition, py::handle x1, py::handle x2, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vc = view_arg(condition, "condition"), *v1 = view_arg(x1, "x1"), *v2 = view_arg(x2, "x2"),
                           *vd = view_arg(dst, "dst");
            if (int rc = dpx_where(vc, v1, v2, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::arg("condition"), py::arg("x1"), py::arg("x2"), py::arg("dst"), py::arg("sycl_queue") = py::none(),
        py::arg("depends") = py::tuple());
    m.def(
        "_where_compare",
        [](int cmp_op, py::handle lhs, py::handle rhs, py::handle x1, py::handle x2, py::handle dst, py::handle sycl_queue,
           py::handle) {
            dpx_array_view *vl = view_arg(lhs, "lhs"), *vr = view_arg(rhs, "rhs"), *v1 = view_arg(x1, "x1"),
                           *v2 = view_arg(x2, "x2"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_where_compare(cmp_op, vl, vr, v1, v2, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::arg("cmp_op"), py::arg("lhs"), py::arg("rhs"), py::arg("x1"), py::arg("x2"), py::arg("dst"),
        py::arg("sycl_queue") = py::none(), py::arg("depends") = py::tuple());
    m.def(
        "_copy_usm_ndarray_into_usm_ndarray",
        [](py::handle src, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vs = view_arg(src, "src"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_copy_cast(vs, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::arg("src"), py::arg("dst"), py::arg("sycl_queue") = py::none(), py::arg("depends") = py::tuple());
    m.def(
        "_divide_by_scalar",
        [](py::handle src, double scalar, py::handle dst, py::handle sycl_queue, py::handle) {
            dpx_array_view *vs = view_arg(src, "src"), *vd = view_arg(dst, "dst");
            if (int rc = dpx_divide_by_scalar(vs, scalar, vd, stream_of(sycl_queue))) raise_status(rc);
            return events_of(sycl_queue);
        },
        py::arg("src"), py::arg("scalar"), py::arg("dst"), py::arg("sycl_queue") = py::none(),
        py::arg("depends") = py::tuple());
    m.def("_array_overlap", [](py::handle a, py::handle b) { return dpx_array_overlap(view_arg(a, "a"), view_arg(b, "b")) != 0; });
    m.def("_same_logical_tensors", [](py::handle a, py::handle b) { return dpx_same_logical(view_arg(a, "a"), view_arg(b, "b")) != 0; });
}
