/* _ti_fastcall: a minimal CPython module that forwards already-validated raw
 * pointers and sizes to the C ABI of libtorch_int_hip.so.  It exists only to
 * cut the per-call cost of ctypes argument conversion (several microseconds,
 * which is more than a decode-sized kernel takes); it has no logic of its own
 * and no dependency on torch. */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>
#include "../../include/torch_int_hip.h"

static inline void* as_ptr(PyObject* o) { return (void*)(uintptr_t)PyLong_AsUnsignedLongLong(o); }
static inline int64_t as_i64(PyObject* o) { return (int64_t)PyLong_AsLongLong(o); }
static inline float as_f32(PyObject* o) { return (float)PyFloat_AsDouble(o); }

/* linear(kind, x, w, bias, out, M, N, K, alpha, beta, ws, ws_bytes, stream) -> status */
static PyObject* fc_linear(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 13) {
    PyErr_SetString(PyExc_TypeError, "linear expects 13 arguments");
    return NULL;
  }
  long kind = PyLong_AsLong(a[0]);
  void *x = as_ptr(a[1]), *w = as_ptr(a[2]), *b = as_ptr(a[3]), *o = as_ptr(a[4]);
  int64_t M = as_i64(a[5]), N = as_i64(a[6]), K = as_i64(a[7]);
  float alpha = as_f32(a[8]), beta = as_f32(a[9]);
  void* ws = as_ptr(a[10]);
  int64_t wsb = as_i64(a[11]);
  void* st = as_ptr(a[12]);
  if (PyErr_Occurred()) return NULL;
  int rc;
  switch (kind) {
    case 0: rc = ti_linear_a8_w8_b32_o32(x, w, b, o, M, N, K, ws, wsb, st); break;
    case 1: rc = ti_linear_a8_w8_b32_o32_with_scaling(x, w, b, o, M, N, K, alpha, beta, ws, wsb, st); break;
    case 2: rc = ti_linear_a8_w8_bfp32_ofp32(x, w, b, o, M, N, K, alpha, beta, ws, wsb, st); break;
    case 3: rc = ti_linear_a8_w8_b8_o8(x, w, b, o, M, N, K, alpha, beta, ws, wsb, st); break;
    case 4: rc = ti_linear_relu_a8_w8_b8_o8(x, w, b, o, M, N, K, alpha, beta, ws, wsb, st); break;
    case 8: rc = ti_linear_a8_w8_bfp32_ofp32_acc(x, w, b, o, M, N, K, alpha, beta, ws, wsb, st); break;
    default:
      PyErr_SetString(PyExc_ValueError, "unknown linear kind");
      return NULL;
  }
  return PyLong_FromLong(rc);
}

/* bmm(kind, a, b, c, batch, M, N, K, alpha, stream) -> status */
static PyObject* fc_bmm(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 10) {
    PyErr_SetString(PyExc_TypeError, "bmm expects 10 arguments");
    return NULL;
  }
  long kind = PyLong_AsLong(a[0]);
  void *pa = as_ptr(a[1]), *pb = as_ptr(a[2]), *pc = as_ptr(a[3]);
  int64_t B = as_i64(a[4]), M = as_i64(a[5]), N = as_i64(a[6]), K = as_i64(a[7]);
  float alpha = as_f32(a[8]);
  void* st = as_ptr(a[9]);
  if (PyErr_Occurred()) return NULL;
  int rc;
  switch (kind) {
    case 5: rc = ti_bmm_s8t_s8n_f32t(pa, pb, pc, B, M, N, K, alpha, st); break;
    case 6: rc = ti_bmm_s8t_s8n_s8t(pa, pb, pc, B, M, N, K, alpha, st); break;
    case 7: rc = ti_bmm_s8t_s8n_s32t(pa, pb, pc, B, M, N, K, st); break;
    default:
      PyErr_SetString(PyExc_ValueError, "unknown bmm kind");
      return NULL;
  }
  return PyLong_FromLong(rc);
}

/* ln_q(input, scale, residual, gamma, beta, eps, r_out, q_out, rows, H, stream) -> status */
static PyObject* fc_ln_q(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 11) {
    PyErr_SetString(PyExc_TypeError, "ln_q expects 11 arguments");
    return NULL;
  }
  void* in = as_ptr(a[0]);
  float scale = as_f32(a[1]);
  void *res = as_ptr(a[2]), *g = as_ptr(a[3]), *b = as_ptr(a[4]);
  float eps = as_f32(a[5]);
  void *ro = as_ptr(a[6]), *qo = as_ptr(a[7]);
  int64_t rows = as_i64(a[8]), H = as_i64(a[9]);
  void* st = as_ptr(a[10]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_dq_add_layernorm_q(in, scale, res, g, b, eps, ro, qo, rows, H, st));
}

/* linear_group3(x, w0, w1, w2, b0, b1, b2, o0, o1, o2, M, N, K, a0, a1, a2, be0, be1, be2, stream) -> status */
static PyObject* fc_linear_group3(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 20) {
    PyErr_SetString(PyExc_TypeError, "linear_group3 expects 20 arguments");
    return NULL;
  }
  const int8_t* x = (const int8_t*)as_ptr(a[0]);
  const int8_t* w[3] = {(const int8_t*)as_ptr(a[1]), (const int8_t*)as_ptr(a[2]), (const int8_t*)as_ptr(a[3])};
  const int8_t* b[3] = {(const int8_t*)as_ptr(a[4]), (const int8_t*)as_ptr(a[5]), (const int8_t*)as_ptr(a[6])};
  int8_t* o[3] = {(int8_t*)as_ptr(a[7]), (int8_t*)as_ptr(a[8]), (int8_t*)as_ptr(a[9])};
  int64_t M = as_i64(a[10]), N = as_i64(a[11]), K = as_i64(a[12]);
  float al[3] = {as_f32(a[13]), as_f32(a[14]), as_f32(a[15])};
  float be[3] = {as_f32(a[16]), as_f32(a[17]), as_f32(a[18])};
  void* st = as_ptr(a[19]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_linear_a8_w8_b8_o8_group(x, w, b, o, al, be, 3, M, N, K, st));
}

/* add_ln_q(x|0, residual, gamma, beta, eps, q_out, rows, H, stream) -> status */
static PyObject* fc_add_ln_q(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 9) {
    PyErr_SetString(PyExc_TypeError, "add_ln_q expects 9 arguments");
    return NULL;
  }
  void *x = as_ptr(a[0]), *res = as_ptr(a[1]), *g = as_ptr(a[2]), *b = as_ptr(a[3]);
  float eps = as_f32(a[4]);
  void* q = as_ptr(a[5]);
  int64_t rows = as_i64(a[6]), H = as_i64(a[7]);
  void* st = as_ptr(a[8]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_add_layernorm_q(x, res, g, b, eps, q, rows, H, st));
}

/* softmax_q(scores, mask|0, probs, batch, heads, T, S, stream) -> status */
static PyObject* fc_softmax_q(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 8) {
    PyErr_SetString(PyExc_TypeError, "softmax_q expects 8 arguments");
    return NULL;
  }
  void *sc = as_ptr(a[0]), *mk = as_ptr(a[1]), *pr = as_ptr(a[2]);
  int64_t B = as_i64(a[3]), Hh = as_i64(a[4]), T = as_i64(a[5]), S = as_i64(a[6]);
  void* st = as_ptr(a[7]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_attn_softmax_q(sc, mk, pr, B, Hh, T, S, st));
}

/* bmm_f32t_strided(a, b, c, batch, M, N, K, stride_a, stride_b, alpha, stream) -> status */
static PyObject* fc_bmm_f32t_strided(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 11) {
    PyErr_SetString(PyExc_TypeError, "bmm_f32t_strided expects 11 arguments");
    return NULL;
  }
  void *pa = as_ptr(a[0]), *pb = as_ptr(a[1]), *pc = as_ptr(a[2]);
  int64_t B = as_i64(a[3]), M = as_i64(a[4]), N = as_i64(a[5]), K = as_i64(a[6]), sa = as_i64(a[7]), sb = as_i64(a[8]);
  float alpha = as_f32(a[9]);
  void* st = as_ptr(a[10]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_bmm_s8t_s8n_f32t_strided(pa, pb, pc, B, M, N, K, sa, sb, alpha, st));
}

/* bmm_rowmajor(a, b, c, batch, M, N, K, stride_b, alpha, stream) -> status */
static PyObject* fc_bmm_rowmajor(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 10) {
    PyErr_SetString(PyExc_TypeError, "bmm_rowmajor expects 10 arguments");
    return NULL;
  }
  void *pa = as_ptr(a[0]), *pb = as_ptr(a[1]), *pc = as_ptr(a[2]);
  int64_t B = as_i64(a[3]), M = as_i64(a[4]), N = as_i64(a[5]), K = as_i64(a[6]), sb = as_i64(a[7]);
  float alpha = as_f32(a[8]);
  void* st = as_ptr(a[9]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_bmm_s8t_s8t_s8t(pa, pb, pc, B, M, N, K, sb, alpha, st));
}

/* kv_append(k_new, v_new, k_buf, v_buf, BH, T, D, cap, S, stream) -> status */
static PyObject* fc_kv_append(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 10) {
    PyErr_SetString(PyExc_TypeError, "kv_append expects 10 arguments");
    return NULL;
  }
  void *kn = as_ptr(a[0]), *vn = as_ptr(a[1]), *kb = as_ptr(a[2]), *vb = as_ptr(a[3]);
  int64_t BH = as_i64(a[4]), T = as_i64(a[5]), D = as_i64(a[6]), cap = as_i64(a[7]), S = as_i64(a[8]);
  void* st = as_ptr(a[9]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_kv_append_s8(kn, vn, kb, vb, BH, T, D, cap, S, st));
}

/* decode_attn(q, k_new, v_new, k_buf, v_buf, mask, ctx, probs, BH, T, D, cap, S, heads, alpha_qk, alpha_pv, stream) -> status */
static PyObject* fc_decode_attn(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 17) {
    PyErr_SetString(PyExc_TypeError, "decode_attn expects 17 arguments");
    return NULL;
  }
  void *q = as_ptr(a[0]), *kn = as_ptr(a[1]), *vn = as_ptr(a[2]), *kb = as_ptr(a[3]), *vb = as_ptr(a[4]);
  void *mask = as_ptr(a[5]), *ctx = as_ptr(a[6]), *probs = as_ptr(a[7]);
  int64_t BH = as_i64(a[8]), T = as_i64(a[9]), D = as_i64(a[10]), cap = as_i64(a[11]), S = as_i64(a[12]);
  int64_t heads = as_i64(a[13]);
  double aqk = PyFloat_AsDouble(a[14]), apv = PyFloat_AsDouble(a[15]);
  void* st = as_ptr(a[16]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_decode_attn_s8(q, kn, vn, kb, vb, mask, ctx, probs, BH, T, D, cap, S, heads, (float)aqk,
                                           (float)apv, st));
}

/* opt_layer_decode(layer, hidden, mask, k_buf, v_buf, B, cap, S, scratch, scratch_bytes, stream) -> status;
 * layer = address of a TiOptDecodeLayer that the caller keeps alive */
static PyObject* fc_opt_layer_decode(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 11) {
    PyErr_SetString(PyExc_TypeError, "opt_layer_decode expects 11 arguments");
    return NULL;
  }
  void *layer = as_ptr(a[0]), *hidden = as_ptr(a[1]), *mask = as_ptr(a[2]), *kb = as_ptr(a[3]), *vb = as_ptr(a[4]);
  int64_t B = as_i64(a[5]), cap = as_i64(a[6]), S = as_i64(a[7]);
  void* scratch = as_ptr(a[8]);
  int64_t sb = as_i64(a[9]);
  void* st = as_ptr(a[10]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_opt_decoder_layer_decode((const TiOptDecodeLayer*)layer, hidden, (const float*)mask, kb, vb, B,
                                                     cap, S, scratch, sb, st));
}

/* opt_layer_prefill(layer, hidden, mask, classes, k_out, v_out, B, T, scratch, scratch_bytes, ws, ws_bytes, stream) -> status */
static PyObject* fc_opt_layer_prefill(PyObject* self, PyObject* const* a, Py_ssize_t n) {
  (void)self;
  if (n != 13) {
    PyErr_SetString(PyExc_TypeError, "opt_layer_prefill expects 13 arguments");
    return NULL;
  }
  void *layer = as_ptr(a[0]), *hidden = as_ptr(a[1]), *mask = as_ptr(a[2]), *cls = as_ptr(a[3]);
  void *ko = as_ptr(a[4]), *vo = as_ptr(a[5]);
  int64_t B = as_i64(a[6]), T = as_i64(a[7]);
  void* scratch = as_ptr(a[8]);
  int64_t sb = as_i64(a[9]);
  void* ws = as_ptr(a[10]);
  int64_t wsb = as_i64(a[11]);
  void* st = as_ptr(a[12]);
  if (PyErr_Occurred()) return NULL;
  return PyLong_FromLong(ti_opt_decoder_layer_prefill((const TiOptDecodeLayer*)layer, hidden, (const float*)mask,
                                                      (const uint8_t*)cls, ko, vo, B, T, scratch, sb, ws, wsb, st));
}

static PyObject* fc_last_error(PyObject* self, PyObject* noargs) {
  (void)self;
  (void)noargs;
  return PyUnicode_FromString(ti_last_error());
}

static PyMethodDef methods[] = {
    {"linear", (PyCFunction)(void (*)(void))fc_linear, METH_FASTCALL, "forward to ti_linear_*"},
    {"bmm", (PyCFunction)(void (*)(void))fc_bmm, METH_FASTCALL, "forward to ti_bmm_*"},
    {"ln_q", (PyCFunction)(void (*)(void))fc_ln_q, METH_FASTCALL, "forward to ti_dq_add_layernorm_q"},
    {"add_ln_q", (PyCFunction)(void (*)(void))fc_add_ln_q, METH_FASTCALL, "forward to ti_add_layernorm_q"},
    {"softmax_q", (PyCFunction)(void (*)(void))fc_softmax_q, METH_FASTCALL, "forward to ti_attn_softmax_q"},
    {"bmm_f32t_strided", (PyCFunction)(void (*)(void))fc_bmm_f32t_strided, METH_FASTCALL, "forward to ti_bmm_s8t_s8n_f32t_strided"},
    {"bmm_rowmajor", (PyCFunction)(void (*)(void))fc_bmm_rowmajor, METH_FASTCALL, "forward to ti_bmm_s8t_s8t_s8t"},
    {"linear_group3", (PyCFunction)(void (*)(void))fc_linear_group3, METH_FASTCALL, "forward to ti_linear_a8_w8_b8_o8_group"},
    {"kv_append", (PyCFunction)(void (*)(void))fc_kv_append, METH_FASTCALL, "forward to ti_kv_append_s8"},
    {"decode_attn", (PyCFunction)(void (*)(void))fc_decode_attn, METH_FASTCALL, "forward to ti_decode_attn_s8"},
    {"opt_layer_decode", (PyCFunction)(void (*)(void))fc_opt_layer_decode, METH_FASTCALL, "forward to ti_opt_decoder_layer_decode"},
    {"opt_layer_prefill", (PyCFunction)(void (*)(void))fc_opt_layer_prefill, METH_FASTCALL, "forward to ti_opt_decoder_layer_prefill"},
    {"last_error", fc_last_error, METH_NOARGS, "ti_last_error()"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef moddef = {PyModuleDef_HEAD_INIT, "_ti_fastcall", "raw-pointer forwarder to libtorch_int_hip.so",
                                    -1, methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__ti_fastcall(void) { return PyModule_Create(&moddef); }
