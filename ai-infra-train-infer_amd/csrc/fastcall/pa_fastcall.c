// A lean way from Python into the C ABI of libpaged_attn.so for the calls a decode step makes
// 140 times: ctypes spends 3-5 us converting the 29 arguments of pa_decode, this module 0.3 us.
// It knows nothing about the library: Python hands it the address of an entry point and the
// entry's argument kinds once (bind), and then calls by index (call).  Nothing is computed here.
//
// Calling convention (x86-64 System V): pointer and integer arguments travel in the integer
// registers and then on the stack, in order; float arguments in the vector registers, in order;
// the two sequences do not interact.  So an entry point `int f(void*, int, long, float, void*)`
// can be called as `f(long, long, long, long, float)`: the integer-class arguments first, widened
// to 64 bits (a callee that takes an `int` reads the low half), then the floats.  Arguments beyond
// those the callee takes are ignored by it (the caller owns the stack), which lets one call site
// with a fixed number of slots serve every signature.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include <stdint.h>
#include <string.h>

#define MAX_BOUND 64
#define MAX_INTS 40
#define MAX_FLOATS 2

typedef struct {
  void* fn;
  char kinds[MAX_INTS + MAX_FLOATS + 1];  // per argument: p pointer (None = null), q int64, i int, f float
  int nargs;
  int wide;  // the entry returns int64 instead of int
} Bound;

static Bound g_bound[MAX_BOUND];
static int g_nbound = 0;

typedef int64_t L;
typedef L (*Entry)(L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L, L,
                   L, L, L, L, L, L, float, float);

// bind(address, kinds, returns_int64) -> index
static PyObject* fc_bind(PyObject* self, PyObject* args) {
  unsigned long long addr;
  const char* kinds;
  int wide;
  if (!PyArg_ParseTuple(args, "Ksp", &addr, &kinds, &wide)) return NULL;
  const size_t n = strlen(kinds);
  int ints = 0, floats = 0;
  for (size_t k = 0; k < n; ++k) {
    if (kinds[k] == 'f') ++floats;
    else if (kinds[k] == 'p' || kinds[k] == 'q' || kinds[k] == 'i') ++ints;
    else {
      PyErr_SetString(PyExc_ValueError, "pa_fastcall.bind: argument kinds are p, q, i and f");
      return NULL;
    }
  }
  if (!addr || ints > MAX_INTS || floats > MAX_FLOATS || g_nbound >= MAX_BOUND) {
    PyErr_SetString(PyExc_ValueError, "pa_fastcall.bind: null address, too many arguments or too many entries");
    return NULL;
  }
  Bound* b = &g_bound[g_nbound];
  b->fn = (void*)(uintptr_t)addr;
  memcpy(b->kinds, kinds, n + 1);
  b->nargs = (int)n;
  b->wide = wide;
  return PyLong_FromLong(g_nbound++);
}

// call(index, *arguments) -> the entry's return value
static PyObject* fc_call(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs < 1) {
    PyErr_SetString(PyExc_TypeError, "pa_fastcall.call: missing the entry's index");
    return NULL;
  }
  const long idx = PyLong_AsLong(args[0]);
  if (idx < 0 || idx >= g_nbound) {
    if (!PyErr_Occurred()) PyErr_SetString(PyExc_IndexError, "pa_fastcall.call: no such entry");
    return NULL;
  }
  const Bound* b = &g_bound[idx];
  if (nargs - 1 != b->nargs) {
    PyErr_Format(PyExc_TypeError, "pa_fastcall.call: the entry takes %d arguments, %zd given", b->nargs, nargs - 1);
    return NULL;
  }
  L a[MAX_INTS];
  float f[MAX_FLOATS] = {0.0f, 0.0f};
  memset(a, 0, sizeof(a));
  int ni = 0, nf = 0;
  for (int k = 0; k < b->nargs; ++k) {
    PyObject* o = args[k + 1];
    switch (b->kinds[k]) {
      case 'p':
        if (o == Py_None) {
          a[ni++] = 0;
        } else if (PyLong_Check(o)) {
          const unsigned long long v = PyLong_AsUnsignedLongLong(o);
          if (v == (unsigned long long)-1 && PyErr_Occurred()) return NULL;
          a[ni++] = (L)v;
        } else {
          PyErr_Format(PyExc_TypeError, "pa_fastcall.call: argument %d must be an address (int) or None", k + 1);
          return NULL;
        }
        break;
      case 'q':
      case 'i': {
        if (!PyLong_Check(o)) {
          PyErr_Format(PyExc_TypeError, "pa_fastcall.call: argument %d must be an int", k + 1);
          return NULL;
        }
        const long long v = PyLong_AsLongLong(o);
        if (v == -1 && PyErr_Occurred()) return NULL;
        if (b->kinds[k] == 'i' && (v < INT32_MIN || v > INT32_MAX)) {
          PyErr_Format(PyExc_OverflowError, "pa_fastcall.call: argument %d does not fit a C int", k + 1);
          return NULL;
        }
        a[ni++] = (L)v;
        break;
      }
      default: {  // 'f'
        const double v = PyFloat_AsDouble(o);
        if (v == -1.0 && PyErr_Occurred()) return NULL;
        f[nf++] = (float)v;
        break;
      }
    }
  }
  L rc;
  Py_BEGIN_ALLOW_THREADS
  rc = ((Entry)b->fn)(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7], a[8], a[9], a[10], a[11], a[12], a[13], a[14], a[15],
                      a[16], a[17], a[18], a[19], a[20], a[21], a[22], a[23], a[24], a[25], a[26], a[27], a[28], a[29],
                      a[30], a[31], a[32], a[33], a[34], a[35], a[36], a[37], a[38], a[39], f[0], f[1]);
  Py_END_ALLOW_THREADS
  return b->wide ? PyLong_FromLongLong(rc) : PyLong_FromLong((long)(int)rc);
}

static PyMethodDef fc_methods[] = {
    {"bind", fc_bind, METH_VARARGS, "bind(address, kinds, returns_int64) -> index of the bound entry"},
    {"call", (PyCFunction)(void (*)(void))fc_call, METH_FASTCALL, "call(index, *arguments) -> the entry's return value"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef fc_module = {PyModuleDef_HEAD_INIT, "pa_fastcall", NULL, -1, fc_methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit_pa_fastcall(void) { return PyModule_Create(&fc_module); }
