// CPython extension `flashlstm._flashlstm`: raw-pointer bindings of the streaming C entry points.
//
// Same calling convention as the reference extension (flashlstm_v2/python/flashlstm/
// _flashlstm_module.cpp:17-103, 105-215): every argument is a Python int -- sizes, device / host
// addresses from tensor.data_ptr(), stream handles from stream.cuda_stream -- 22 of them for
// forward and 30 for backward, in the order listed below; 0 stands for a null pointer.  The GIL is
// released while the library runs.  Both functions return None.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include "flashlstm_v2/lstm.hpp"

namespace {

template <typename T>
T* as_ptr(unsigned long long v) { return reinterpret_cast<T*>(static_cast<uintptr_t>(v)); }

hipStream_t as_stream(unsigned long long v) { return reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(v)); }

bool parse_ints(PyObject* args, const char* name, unsigned long long* out, Py_ssize_t n) {
    if (!PyTuple_Check(args) || PyTuple_GET_SIZE(args) != n) {
        PyErr_Format(PyExc_TypeError, "%s expects exactly %zd integer arguments (got %zd)", name, n,
                     PyTuple_Check(args) ? PyTuple_GET_SIZE(args) : (Py_ssize_t)-1);
        return false;
    }
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject* item = PyTuple_GET_ITEM(args, i);
        if (!PyLong_Check(item)) {
            PyErr_Format(PyExc_TypeError, "%s: argument %zd must be an int", name, i + 1);
            return false;
        }
        out[i] = PyLong_AsUnsignedLongLongMask(item);
        if (PyErr_Occurred()) return false;
    }
    return true;
}

// T, B, I, H, R, x_host, h0, c0, W_ih, W_hh, b_ih, b_hh, y_host, cache_h, cache_c, cache_h_dtype,
// cache_c_dtype, hy, cy, compute_stream, h2d_stream, d2h_stream
PyObject* streaming_lstm_forward(PyObject*, PyObject* args) {
    unsigned long long a[22];
    if (!parse_ints(args, "streaming_lstm_forward", a, 22)) return nullptr;
    flstm_GateCacheHost cache{as_ptr<void>(a[13]), as_ptr<void>(a[14])};
    flstm_StreamingLstmOptions opt{static_cast<flstm_GateCacheDType>(a[15]), static_cast<flstm_GateCacheDType>(a[16])};
    Py_BEGIN_ALLOW_THREADS
    flstm_StreamingLstmForward(a[0], a[1], a[2], a[3], a[4], as_ptr<const __half>(a[5]), as_ptr<const __half>(a[6]),
                               as_ptr<const __half>(a[7]), as_ptr<const float>(a[8]), as_ptr<const float>(a[9]),
                               as_ptr<const float>(a[10]), as_ptr<const float>(a[11]), as_ptr<__half>(a[12]), cache,
                               &opt, as_ptr<__half>(a[17]), as_ptr<__half>(a[18]), as_stream(a[19]), as_stream(a[20]),
                               as_stream(a[21]));
    Py_END_ALLOW_THREADS
    Py_RETURN_NONE;
}

// T, B, I, H, R, x_host, y_host, cache_h, cache_c, cache_h_dtype, cache_c_dtype, dY_host, d_hn, d_cn,
// h0, c0, W_ih, W_hh, b_ih, b_hh, dx_host, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, compute_stream,
// h2d_stream, d2h_stream
PyObject* streaming_lstm_backward(PyObject*, PyObject* args) {
    unsigned long long a[30];
    if (!parse_ints(args, "streaming_lstm_backward", a, 30)) return nullptr;
    flstm_GateCacheHost cache{as_ptr<void>(a[7]), as_ptr<void>(a[8])};
    flstm_StreamingLstmOptions opt{static_cast<flstm_GateCacheDType>(a[9]), static_cast<flstm_GateCacheDType>(a[10])};
    Py_BEGIN_ALLOW_THREADS
    flstm_StreamingLstmBackward(a[0], a[1], a[2], a[3], a[4], as_ptr<const __half>(a[5]), as_ptr<const __half>(a[6]),
                                cache, as_ptr<const __half>(a[11]), as_ptr<const __half>(a[12]),
                                as_ptr<const __half>(a[13]), as_ptr<const __half>(a[14]), as_ptr<const __half>(a[15]),
                                as_ptr<const float>(a[16]), as_ptr<const float>(a[17]), as_ptr<const float>(a[18]),
                                as_ptr<const float>(a[19]), as_ptr<__half>(a[20]), as_ptr<float>(a[21]),
                                as_ptr<float>(a[22]), as_ptr<float>(a[23]), as_ptr<float>(a[24]), as_ptr<float>(a[25]),
                                as_ptr<float>(a[26]), as_stream(a[27]), as_stream(a[28]), as_stream(a[29]), &opt);
    Py_END_ALLOW_THREADS
    Py_RETURN_NONE;
}

PyObject* release_caches(PyObject*, PyObject*) {
    flstm_ReleaseStreamingCaches();
    Py_RETURN_NONE;
}

PyMethodDef kMethods[] = {
    {"streaming_lstm_forward", streaming_lstm_forward, METH_VARARGS,
     "streaming_lstm_forward(T, B, I, H, R, x_host, h0, c0, W_ih, W_hh, b_ih, b_hh, y_host, cache_h, cache_c, "
     "cache_h_dtype, cache_c_dtype, hy, cy, compute_stream, h2d_stream, d2h_stream) -> None"},
    {"streaming_lstm_backward", streaming_lstm_backward, METH_VARARGS,
     "streaming_lstm_backward(T, B, I, H, R, x_host, y_host, cache_h, cache_c, cache_h_dtype, cache_c_dtype, "
     "dY_host, d_hn, d_cn, h0, c0, W_ih, W_hh, b_ih, b_hh, dx_host, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, "
     "compute_stream, h2d_stream, d2h_stream) -> None"},
    {"release_caches", release_caches, METH_NOARGS, "Free device buffers kept between calls."},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef kModule = {PyModuleDef_HEAD_INIT, "_flashlstm",
                       "Raw bindings of the MI355X streaming LSTM kernels.", -1, kMethods,
                       nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__flashlstm(void) { return PyModule_Create(&kModule); }
