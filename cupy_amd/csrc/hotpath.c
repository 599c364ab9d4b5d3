/* CPython extension for the calls the host makes per kernel launch:
 * the signature of its arguments (the key a recorded call is found by), the
 * launch itself, the replay of a recorded call, and the memory pool's
 * malloc/free.  Each is a thin caller of the C-ABI in include/mi355rt.h
 * (rt_launch_packed, rt_pool_malloc, rt_pool_free); what it removes is the
 * per-argument conversion cost of a ctypes call (about 1 us for the eleven
 * arguments of a launch) and the interpreter loop that splices pointers into a
 * recorded argument block.  The reference does this part of the path in
 * compiled Cython (cupy/_core/_kernel.pyx:166-247 argument packing,
 * cupy/cuda/function.pyx:191-236 launch, cupy/cuda/memory.pyx:1373-1441 pool).
 *
 * Nothing here touches the GPU on its own: every GPU effect goes through the
 * C-ABI, so the library and this module cannot disagree about it.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>
#include <string.h>

#include "mi355rt.h"

static PyObject* str_data;
static PyObject* str_ptr;
static PyObject* str_dtype;
static PyObject* str_shape;
static PyObject* str_strides;
static PyObject* str_device_id;
static PyTypeObject* array_type;      /* the package's ndarray, set by setup() */
static PyTypeObject* generic_type;    /* numpy.generic */

static int as_u64(PyObject* o, uint64_t* out) {
  unsigned long long v = PyLong_AsUnsignedLongLong(o);
  if (v == (unsigned long long)-1 && PyErr_Occurred()) return -1;
  *out = (uint64_t)v;
  return 0;
}

static int as_u32(PyObject* o, unsigned* out) {
  unsigned long v = PyLong_AsUnsignedLong(o);
  if (v == (unsigned long)-1 && PyErr_Occurred()) return -1;
  if (v > 0xfffffffful) {
    PyErr_SetString(PyExc_OverflowError, "launch dimension does not fit 32 bits");
    return -1;
  }
  *out = (unsigned)v;
  return 0;
}

/* launch(function, gx, gy, gz, bx, by, bz, shared_mem, stream, arg_block) -> status */
static PyObject* hp_launch(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 10) {
    PyErr_SetString(PyExc_TypeError, "launch takes 10 arguments");
    return NULL;
  }
  uint64_t fn, stream;
  unsigned d[7];
  if (as_u64(args[0], &fn) < 0) return NULL;
  for (int i = 0; i < 7; ++i)
    if (as_u32(args[1 + i], &d[i]) < 0) return NULL;
  if (as_u64(args[8], &stream) < 0) return NULL;
  Py_buffer view;
  if (PyObject_GetBuffer(args[9], &view, PyBUF_SIMPLE) < 0) return NULL;
  int status;
  Py_BEGIN_ALLOW_THREADS
  status = rt_launch_packed((void*)(uintptr_t)fn, d[0], d[1], d[2], d[3], d[4], d[5], d[6],
                            (void*)(uintptr_t)stream, view.buf, (size_t)view.len);
  Py_END_ALLOW_THREADS
  PyBuffer_Release(&view);
  return PyLong_FromLong(status);
}

/* A recorded call, as one bytes object:
 *   u32 n_launches, u32 0
 *   per launch (8-byte aligned):
 *     u64 function, u32 grid[3], u32 block[3], u32 shared_mem, u32 n_slots,
 *     u64 block_size, then n_slots x (u32 byte offset, u32 ref), padded to 8,
 *     then the argument block, padded to 8.
 * A slot names the 8 bytes of the block that receive the device address of
 * refs[ref]: of its `.data.ptr` for ref < n_arrays (an array), of its `.ptr`
 * otherwise (a temporary's memory pointer). */
typedef struct {
  uint64_t function;
  uint32_t grid[3];
  uint32_t block[3];
  uint32_t shared_mem;
  uint32_t n_slots;
  uint64_t block_size;
} LaunchHeader;

#define HP_STACK_BLOCK 4096

static int address_of(PyObject* ref, int is_array, uint64_t* out) {
  PyObject* holder = ref;
  PyObject* data = NULL;
  if (is_array) {
    data = PyObject_GetAttr(ref, str_data);
    if (!data) return -1;
    holder = data;
  }
  PyObject* ptr = PyObject_GetAttr(holder, str_ptr);
  Py_XDECREF(data);
  if (!ptr) return -1;
  int rc = as_u64(ptr, out);
  Py_DECREF(ptr);
  return rc;
}

/* Walks a launch record: patches every argument block and either launches it
 * (`listing` NULL; returns the first non-zero status as an int object, else 0)
 * or appends (function, grid, block, shared_mem, patched block) to `listing`. */
static PyObject* walk_record(PyObject* record, PyObject* refs, long n_arrays, uint64_t stream,
                             PyObject* listing) {
  const unsigned char* rec = (const unsigned char*)PyBytes_AS_STRING(record);
  const size_t rec_size = (size_t)PyBytes_GET_SIZE(record);
  const Py_ssize_t n_refs = PyList_GET_SIZE(refs);
  unsigned char stack_block[HP_STACK_BLOCK] __attribute__((aligned(16)));
  uint32_t n_launches;
  size_t pos = 8;
  if (rec_size < 8) goto malformed;
  memcpy(&n_launches, rec, 4);
  for (uint32_t l = 0; l < n_launches; ++l) {
    LaunchHeader h;
    if (pos + sizeof(h) > rec_size) goto malformed;
    memcpy(&h, rec + pos, sizeof(h));
    pos += sizeof(h);
    const size_t slot_bytes = ((size_t)h.n_slots * 8 + 7) & ~(size_t)7;
    const size_t block_bytes = ((size_t)h.block_size + 7) & ~(size_t)7;
    if (slot_bytes > rec_size || block_bytes > rec_size ||
        pos + slot_bytes + block_bytes > rec_size)
      goto malformed;
    const unsigned char* slots = rec + pos;
    pos += slot_bytes;
    unsigned char* block = stack_block;
    if (h.block_size > HP_STACK_BLOCK) {
      block = (unsigned char*)PyMem_Malloc((size_t)h.block_size);
      if (!block) return PyErr_NoMemory();
    }
    memcpy(block, rec + pos, (size_t)h.block_size);
    pos += block_bytes;
    int bad = 0;
    for (uint32_t s = 0; s < h.n_slots; ++s) {
      uint32_t off, ref;
      memcpy(&off, slots + 8 * s, 4);
      memcpy(&ref, slots + 8 * s + 4, 4);
      if ((size_t)off + 8 > h.block_size || (Py_ssize_t)ref >= n_refs) {
        bad = 2;
        break;
      }
      uint64_t address;
      if (address_of(PyList_GET_ITEM(refs, ref), (long)ref < n_arrays, &address) < 0) {
        bad = 1;
        break;
      }
      memcpy(block + off, &address, 8);
    }
    int status = 0;
    if (!bad && listing) {
      PyObject* entry = Py_BuildValue(
          "K(III)(III)Iy#", (unsigned long long)h.function, h.grid[0], h.grid[1], h.grid[2],
          h.block[0], h.block[1], h.block[2], h.shared_mem, (const char*)block,
          (Py_ssize_t)h.block_size);
      if (!entry || PyList_Append(listing, entry) < 0) bad = 1;
      Py_XDECREF(entry);
    } else if (!bad) {
      Py_BEGIN_ALLOW_THREADS
      status = rt_launch_packed((void*)(uintptr_t)h.function, h.grid[0], h.grid[1], h.grid[2],
                                h.block[0], h.block[1], h.block[2], h.shared_mem,
                                (void*)(uintptr_t)stream, block, (size_t)h.block_size);
      Py_END_ALLOW_THREADS
    }
    if (block != stack_block) PyMem_Free(block);
    if (bad == 1) return NULL;
    if (bad == 2) goto malformed;
    if (status != 0) return PyLong_FromLong(status);
  }
  return PyLong_FromLong(0);
malformed:
  PyErr_SetString(PyExc_ValueError, "malformed launch record");
  return NULL;
}

/* replay(record, refs, n_arrays, stream) -> status of the first launch that failed, or 0 */
static PyObject* hp_replay(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 4 || !PyBytes_Check(args[0]) || !PyList_Check(args[1])) {
    PyErr_SetString(PyExc_TypeError, "replay(record: bytes, refs: list, n_arrays, stream)");
    return NULL;
  }
  const long n_arrays = PyLong_AsLong(args[2]);
  if (n_arrays == -1 && PyErr_Occurred()) return NULL;
  uint64_t stream;
  if (as_u64(args[3], &stream) < 0) return NULL;
  return walk_record(args[0], args[1], n_arrays, stream, NULL);
}

/* splice(record, refs, n_arrays) -> [(function, grid, block, shared_mem, argument block)]:
 * what replay() would launch, without launching it */
static PyObject* hp_splice(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 3 || !PyBytes_Check(args[0]) || !PyList_Check(args[1])) {
    PyErr_SetString(PyExc_TypeError, "splice(record: bytes, refs: list, n_arrays)");
    return NULL;
  }
  const long n_arrays = PyLong_AsLong(args[2]);
  if (n_arrays == -1 && PyErr_Occurred()) return NULL;
  PyObject* listing = PyList_New(0);
  if (!listing) return NULL;
  PyObject* status = walk_record(args[0], args[1], n_arrays, 0, listing);
  if (!status) {
    Py_DECREF(listing);
    return NULL;
  }
  Py_DECREF(status);
  return listing;
}

/* pool_malloc(pool, size, stream_ident) -> address, or -status on failure */
static PyObject* hp_pool_malloc(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 3) {
    PyErr_SetString(PyExc_TypeError, "pool_malloc takes 3 arguments");
    return NULL;
  }
  uint64_t pool, size, ident, address = 0;
  if (as_u64(args[0], &pool) < 0 || as_u64(args[1], &size) < 0 || as_u64(args[2], &ident) < 0)
    return NULL;
  int status;
  /* the pool may call back into Python (a user's allocator) and may wait for
   * another thread that does: the interpreter lock must not be held */
  Py_BEGIN_ALLOW_THREADS
  status = rt_pool_malloc((void*)(uintptr_t)pool, (size_t)size, ident, &address);
  Py_END_ALLOW_THREADS
  if (status != 0) return PyLong_FromLong(-(long)status);
  return PyLong_FromUnsignedLongLong(address);
}

/* pool_free(pool, address) -> status */
static PyObject* hp_pool_free(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 2) {
    PyErr_SetString(PyExc_TypeError, "pool_free takes 2 arguments");
    return NULL;
  }
  uint64_t pool, address;
  if (as_u64(args[0], &pool) < 0 || as_u64(args[1], &address) < 0) return NULL;
  int status;
  Py_BEGIN_ALLOW_THREADS
  status = rt_pool_free((void*)(uintptr_t)pool, address);
  Py_END_ALLOW_THREADS
  return PyLong_FromLong(status);
}

/* get_device() -> index of the calling thread's current device, or -status */
static PyObject* hp_get_device(PyObject* self, PyObject* unused) {
  (void)self;
  (void)unused;
  int device = 0;
  int status = rt_get_device(&device);
  if (status != 0) return PyLong_FromLong(-(long)status);
  return PyLong_FromLong(device);
}

/* setup(ndarray type, numpy.generic) */
static PyObject* hp_setup(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 2 || !PyType_Check(args[0]) || !PyType_Check(args[1])) {
    PyErr_SetString(PyExc_TypeError, "setup(array type, numpy.generic)");
    return NULL;
  }
  Py_INCREF(args[0]);
  Py_INCREF(args[1]);
  Py_XDECREF((PyObject*)array_type);
  Py_XDECREF((PyObject*)generic_type);
  array_type = (PyTypeObject*)args[0];
  generic_type = (PyTypeObject*)args[1];
  Py_RETURN_NONE;
}

/* One array's part of a call signature: (dtype, shape, strides, address & 15),
 * or NULL with no error set if the array lives on another device. */
static PyObject* array_signature(PyObject* a, PyObject* dev_id) {
  PyObject *data = NULL, *dev = NULL, *ptr = NULL, *dtype = NULL, *shape = NULL, *strides = NULL;
  PyObject *low = NULL, *out = NULL;
  data = PyObject_GetAttr(a, str_data);
  if (!data) goto done;
  dev = PyObject_GetAttr(data, str_device_id);
  if (!dev) goto done;
  int same = PyObject_RichCompareBool(dev, dev_id, Py_EQ);
  if (same <= 0) goto done;           /* another device (no error) or a failed comparison */
  ptr = PyObject_GetAttr(data, str_ptr);
  if (!ptr) goto done;
  uint64_t address;
  if (as_u64(ptr, &address) < 0) goto done;
  dtype = PyObject_GetAttr(a, str_dtype);
  shape = PyObject_GetAttr(a, str_shape);
  strides = PyObject_GetAttr(a, str_strides);
  low = PyLong_FromLong((long)(address & 15));
  if (!dtype || !shape || !strides || !low) goto done;
  out = PyTuple_Pack(4, dtype, shape, strides, low);
done:
  Py_XDECREF(data);
  Py_XDECREF(dev);
  Py_XDECREF(ptr);
  Py_XDECREF(dtype);
  Py_XDECREF(shape);
  Py_XDECREF(strides);
  Py_XDECREF(low);
  return out;
}

/* signature(args: tuple or list, device id, tuning version) -> tuple, or None when the
 * call must take the full path: everything about the arguments that launch
 * decisions may depend on.  Arrays contribute (dtype, shape, strides,
 * alignment of the address), scalars their type. */
static PyObject* hp_signature(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 3 || !(PyTuple_Check(args[0]) || PyList_Check(args[0]))) {
    PyErr_SetString(PyExc_TypeError, "signature(args: tuple or list, device id, version)");
    return NULL;
  }
  if (!array_type) {
    PyErr_SetString(PyExc_RuntimeError, "signature: setup() has not been called");
    return NULL;
  }
  PyObject* call = args[0];
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(call);
  PyObject* sig = PyTuple_New(n + 2);
  if (!sig) return NULL;
  Py_INCREF(args[1]);
  PyTuple_SET_ITEM(sig, 0, args[1]);
  Py_INCREF(args[2]);
  PyTuple_SET_ITEM(sig, 1, args[2]);
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject* a = PySequence_Fast_GET_ITEM(call, i);
    PyTypeObject* t = Py_TYPE(a);
    PyObject* item = NULL;
    if (t == array_type) {
      item = array_signature(a, args[1]);
      if (!item) {
        Py_DECREF(sig);
        if (PyErr_Occurred()) return NULL;
        Py_RETURN_NONE;
      }
    } else if (t == &PyFloat_Type || t == &PyBool_Type || t == &PyComplex_Type) {
      item = (PyObject*)t;
      Py_INCREF(item);
    } else if (t == &PyLong_Type) {
      int overflow = 0;
      (void)PyLong_AsLongLongAndOverflow(a, &overflow);
      if (overflow) {
        Py_DECREF(sig);
        Py_RETURN_NONE;
      }
      item = (PyObject*)t;
      Py_INCREF(item);
    } else if (PyType_IsSubtype(t, generic_type)) {
      item = (PyObject*)t;
      Py_INCREF(item);
    } else {
      Py_DECREF(sig);
      Py_RETURN_NONE;
    }
    PyTuple_SET_ITEM(sig, i + 2, item);
  }
  return sig;
}

static PyMethodDef methods[] = {
    {"get_device", hp_get_device, METH_NOARGS, "get_device() -> device index or -status"},
    {"setup", (PyCFunction)(void (*)(void))hp_setup, METH_FASTCALL,
     "setup(array type, numpy.generic)"},
    {"signature", (PyCFunction)(void (*)(void))hp_signature, METH_FASTCALL,
     "signature(args, device id, version) -> tuple or None"},
    {"launch", (PyCFunction)(void (*)(void))hp_launch, METH_FASTCALL,
     "launch(function, gx, gy, gz, bx, by, bz, shared_mem, stream, arg_block) -> status"},
    {"replay", (PyCFunction)(void (*)(void))hp_replay, METH_FASTCALL,
     "replay(record, refs, n_arrays, stream) -> status"},
    {"splice", (PyCFunction)(void (*)(void))hp_splice, METH_FASTCALL,
     "splice(record, refs, n_arrays) -> list of launches as replay() would make them"},
    {"pool_malloc", (PyCFunction)(void (*)(void))hp_pool_malloc, METH_FASTCALL,
     "pool_malloc(pool, size, stream_ident) -> address or -status"},
    {"pool_free", (PyCFunction)(void (*)(void))hp_pool_free, METH_FASTCALL,
     "pool_free(pool, address) -> status"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_hotpath",
                                    "Per-launch host calls of cupy_amd in C.", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__hotpath(void) {
  str_data = PyUnicode_InternFromString("data");
  str_ptr = PyUnicode_InternFromString("ptr");
  str_dtype = PyUnicode_InternFromString("dtype");
  str_shape = PyUnicode_InternFromString("_shape");
  str_strides = PyUnicode_InternFromString("_strides");
  str_device_id = PyUnicode_InternFromString("device_id");
  if (!str_data || !str_ptr || !str_dtype || !str_shape || !str_strides || !str_device_id)
    return NULL;
  return PyModule_Create(&module);
}
