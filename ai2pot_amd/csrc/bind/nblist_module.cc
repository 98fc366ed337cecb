// CPython extension module `nblist` with the reference module's single function
//   find_info4mlff(lattice, types, coords, rcut, umax, is_cart, pbc_xyz, sort)
//       -> (inum, ilist, numneigh, firstneigh, rcs, types, nghost)
// (source/nblist/bind/nblist_bind.cc:35-207): same positional signature, same type checks
// (TypeError), NumPy arrays in and out, float32 / float64 selected by the dtype of coords.
// The list is built on the current HIP device by libai2pot_hip.so; inputs are copied to the
// device and results back.  Unlike the reference, more than `umax` neighbours raises
// RuntimeError instead of overrunning the output arrays.
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#define NPY_NO_DEPRECATED_API NPY_1_7_API_VERSION
#include <numpy/arrayobject.h>
#include <hip/hip_runtime_api.h>

#include <string>
#include <vector>

#include "../../../include/ai2pot_hip.h"

namespace {

struct DeviceBuf {
    void* p = nullptr;
    ~DeviceBuf() { if (p) (void)hipFree(p); }
    bool alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess; }
};

PyObject* fail(PyObject* exc, const std::string& msg)
{
    PyErr_SetString(exc, msg.c_str());
    return nullptr;
}

template <typename T>
PyObject* run(PyArrayObject* lattice, PyArrayObject* types, PyArrayObject* coords, double rcut, int umax,
              bool is_cart, const int* pbc, bool sort, int npy_float)
{
    const int n = (int)PyArray_DIM(coords, 0);
    if (n <= 0) return fail(PyExc_RuntimeError, "the structure has no atoms");
    DeviceBuf d_types, d_coords, d_ilist, d_nn, d_first, d_rcs, d_tout;
    const size_t row = (size_t)n * umax;
    if (!d_types.alloc(sizeof(int) * n) || !d_coords.alloc(sizeof(T) * n * 3) || !d_ilist.alloc(sizeof(int) * n) ||
        !d_nn.alloc(sizeof(int) * n) || !d_first.alloc(sizeof(int) * row) || !d_rcs.alloc(sizeof(T) * row * 3) ||
        !d_tout.alloc(sizeof(int) * n))
        return fail(PyExc_MemoryError, "hipMalloc failed");
    if (hipMemcpy(d_types.p, PyArray_DATA(types), sizeof(int) * n, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(d_coords.p, PyArray_DATA(coords), sizeof(T) * n * 3, hipMemcpyHostToDevice) != hipSuccess)
        return fail(PyExc_RuntimeError, "copy to the device failed");
    int max_nn = 0, rc;
    if (sizeof(T) == 4)
        rc = a2p_nblist_build_f32((const float*)PyArray_DATA(lattice), (const int*)d_types.p,
                                  (const float*)d_coords.p, n, rcut, umax, is_cart, pbc, sort, (int*)d_ilist.p,
                                  (int*)d_nn.p, (int*)d_first.p, (float*)d_rcs.p, (int*)d_tout.p, &max_nn, nullptr);
    else
        rc = a2p_nblist_build_f64((const double*)PyArray_DATA(lattice), (const int*)d_types.p,
                                  (const double*)d_coords.p, n, rcut, umax, is_cart, pbc, sort, (int*)d_ilist.p,
                                  (int*)d_nn.p, (int*)d_first.p, (double*)d_rcs.p, (int*)d_tout.p, &max_nn, nullptr);
    if (rc != A2P_OK) return fail(PyExc_RuntimeError, std::string("libai2pot_hip: ") + a2p_last_error());

    npy_intp d1[1] = {n}, d2[2] = {n, umax}, d3[3] = {n, umax, 3};
    PyObject* ilist = PyArray_SimpleNew(1, d1, NPY_INT32);
    PyObject* nn = PyArray_SimpleNew(1, d1, NPY_INT32);
    PyObject* first = PyArray_SimpleNew(2, d2, NPY_INT32);
    PyObject* rcs = PyArray_SimpleNew(3, d3, npy_float);
    PyObject* tout = PyArray_SimpleNew(1, d1, NPY_INT32);
    bool ok = ilist && nn && first && rcs && tout;
    ok = ok && hipMemcpy(PyArray_DATA((PyArrayObject*)ilist), d_ilist.p, sizeof(int) * n, hipMemcpyDeviceToHost) == hipSuccess;
    ok = ok && hipMemcpy(PyArray_DATA((PyArrayObject*)nn), d_nn.p, sizeof(int) * n, hipMemcpyDeviceToHost) == hipSuccess;
    ok = ok && hipMemcpy(PyArray_DATA((PyArrayObject*)first), d_first.p, sizeof(int) * row, hipMemcpyDeviceToHost) == hipSuccess;
    ok = ok && hipMemcpy(PyArray_DATA((PyArrayObject*)rcs), d_rcs.p, sizeof(T) * row * 3, hipMemcpyDeviceToHost) == hipSuccess;
    ok = ok && hipMemcpy(PyArray_DATA((PyArrayObject*)tout), d_tout.p, sizeof(int) * n, hipMemcpyDeviceToHost) == hipSuccess;
    if (!ok) {
        Py_XDECREF(ilist); Py_XDECREF(nn); Py_XDECREF(first); Py_XDECREF(rcs); Py_XDECREF(tout);
        return fail(PyExc_RuntimeError, "copy from the device failed");
    }
    return Py_BuildValue("(iNNNNNi)", n, ilist, nn, first, rcs, tout, 0);
}

PyObject* py_find_info4mlff(PyObject*, PyObject* args)
{
    PyObject *lat, *types_in, *coords, *rcut, *umax, *is_cart, *pbc, *sort;
    if (!PyArg_ParseTuple(args, "OOOOOOOO", &lat, &types_in, &coords, &rcut, &umax, &is_cart, &pbc, &sort))
        return nullptr;
    if (!PyArray_Check(lat) || !PyArray_Check(types_in) || !PyArray_Check(coords) || !PyFloat_Check(rcut) ||
        !PyLong_Check(umax) || PyBool_Check(umax) || !PyBool_Check(is_cart) || !PyList_Check(pbc) ||
        !PyBool_Check(sort))
        return fail(PyExc_TypeError, "Please check the parameter in interface of py_find_info4mlff().");
    if (PyList_Size(pbc) != 3) return fail(PyExc_TypeError, "pbc_xyz must have three entries");
    const int ft = PyArray_TYPE((PyArrayObject*)coords);
    if ((ft != NPY_FLOAT32 && ft != NPY_FLOAT64) || PyArray_TYPE((PyArrayObject*)lat) != ft)
        return fail(PyExc_TypeError, "lattice and coords must share dtype float32 or float64");
    const int it = PyArray_TYPE((PyArrayObject*)types_in);
    if (it != NPY_INT32 && it != NPY_INT64) return fail(PyExc_TypeError, "types must be int32 or int64");
    if (PyArray_NDIM((PyArrayObject*)coords) != 2 || PyArray_DIM((PyArrayObject*)coords, 1) != 3 ||
        PyArray_SIZE((PyArrayObject*)lat) != 9 ||
        PyArray_SIZE((PyArrayObject*)types_in) != PyArray_DIM((PyArrayObject*)coords, 0))
        return fail(PyExc_TypeError, "expected lattice[3,3], types[N], coords[N,3]");
    // the reference reads the raw buffers (C order); make that explicit instead of assuming it
    PyArrayObject* c_lat = (PyArrayObject*)PyArray_FROM_OTF(lat, ft, NPY_ARRAY_IN_ARRAY);
    PyArrayObject* c_coords = (PyArrayObject*)PyArray_FROM_OTF(coords, ft, NPY_ARRAY_IN_ARRAY);
    PyArrayObject* c_types = (PyArrayObject*)PyArray_FROM_OTF(types_in, NPY_INT32, NPY_ARRAY_IN_ARRAY | NPY_ARRAY_FORCECAST);
    if (!c_lat || !c_coords || !c_types) {
        Py_XDECREF(c_lat); Py_XDECREF(c_coords); Py_XDECREF(c_types);
        return nullptr;
    }
    int pbc_i[3];
    for (int i = 0; i < 3; i++) pbc_i[i] = PyObject_IsTrue(PyList_GetItem(pbc, i)) ? 1 : 0;
    const long umax_l = PyLong_AsLong(umax);
    PyObject* out;
    if (umax_l <= 0 || umax_l > (1 << 20)) out = fail(PyExc_RuntimeError, "umax must be positive");
    else if (ft == NPY_FLOAT32)
        out = run<float>(c_lat, c_types, c_coords, PyFloat_AsDouble(rcut), (int)umax_l, PyObject_IsTrue(is_cart),
                         pbc_i, PyObject_IsTrue(sort), NPY_FLOAT32);
    else
        out = run<double>(c_lat, c_types, c_coords, PyFloat_AsDouble(rcut), (int)umax_l, PyObject_IsTrue(is_cart),
                          pbc_i, PyObject_IsTrue(sort), NPY_FLOAT64);
    Py_DECREF(c_lat); Py_DECREF(c_coords); Py_DECREF(c_types);
    return out;
}

PyMethodDef methods[] = {
    {"find_info4mlff", (PyCFunction)&py_find_info4mlff, METH_VARARGS, "nblist.find_info4mlff() on the GPU"},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef moddef = {PyModuleDef_HEAD_INIT, "nblist", "periodic neighbour list (libai2pot_hip)", -1, methods};

}  // namespace

PyMODINIT_FUNC PyInit_nblist(void)
{
    import_array();
    return PyModule_Create(&moddef);
}
