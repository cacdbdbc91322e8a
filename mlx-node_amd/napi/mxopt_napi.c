/* N-API binding of libmxopt.so: the JavaScript surface of the reference for this path
 * (packages/core/index.d.cts: Adam :38-56, AdamW :66-81, SGD :1855-1872, RMSprop :1696-1712,
 * GradientUtils :486-521, LRScheduler :722-750, clipGradientsByGlobalNorm :2144,
 * clipGradientsByValue :2159, Qwen3Model.accumulateGradients :1315, DType :2304-2310) with the same
 * class names, method names, argument order, defaults and error codes, over a small MxArray that
 * owns a device buffer (fromFloat32 / zeros / toFloat32 / shape / size / dtype / astype only).
 *
 * The reference generates its binding from Rust with napi-rs; this one is hand-written C against
 * node_api.h so that it builds with the toolchain that is present (node 12, gcc).  Every method is a
 * shim: unwrap the arrays, allocate the result array the reference would have returned, call the
 * C ABI.  Errors become JS exceptions whose `code` is "InvalidArg" or "GenericFailure", as napi-rs
 * sets it (crates/mlx-core/src/optimizers/sgd.rs:51-56).
 */
#define NAPI_VERSION 6
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <node_api.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "mxopt_engine.h"

static mxopt_ctx* g_ctx;
static napi_ref g_array_ctor;

typedef struct {
  void* data;
  uint64_t n;
  int dtype;
  int ndim;
  int64_t shape[8];
} Array;

typedef struct {
  mxopt_optimizer* opt;
} Optimizer;

/* ---- errors ------------------------------------------------------------------------ */

static napi_value throw_code(napi_env env, const char* code, const char* msg) {
  napi_throw_error(env, code, msg);
  return NULL;
}

static napi_value throw_status(napi_env env, int rc) {
  return throw_code(env, rc == MXOPT_ERR_INVALID_ARG ? "InvalidArg" : "GenericFailure", mxopt_last_error(g_ctx));
}

#define NAPI_OK(call)                                                             \
  do {                                                                            \
    if ((call) != napi_ok) return throw_code(env, "GenericFailure", "N-API call failed: " #call); \
  } while (0)
#define MX_OK(call)                                   \
  do {                                                \
    int rc_ = (call);                                 \
    if (rc_ != MXOPT_OK) return throw_status(env, rc_); \
  } while (0)

/* ---- MxArray ----------------------------------------------------------------------- */

static void array_finalize(napi_env env, void* data, void* hint) {
  (void)env; (void)hint;
  Array* a = (Array*)data;
  if (a->data) {
    (void)mxopt_synchronize(g_ctx); /* a kernel may still be reading the buffer */
    (void)hipFree(a->data);
  }
  free(a);
}

static napi_value array_construct(napi_env env, napi_callback_info info) {
  napi_value self;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Array* a = (Array*)calloc(1, sizeof *a);
  if (!a) return throw_code(env, "GenericFailure", "out of memory");
  NAPI_OK(napi_wrap(env, self, a, array_finalize, NULL, NULL));
  return self;
}

static int dtype_bytes(int dt) { return dt == MXOPT_F32 ? 4 : 2; }

/* A new array of `n` elements; shape copied from `like` when given, else [n]. */
static napi_value new_array(napi_env env, uint64_t n, int dtype, const Array* like, Array** out) {
  napi_value ctor, obj;
  NAPI_OK(napi_get_reference_value(env, g_array_ctor, &ctor));
  NAPI_OK(napi_new_instance(env, ctor, 0, NULL, &obj));
  Array* a;
  NAPI_OK(napi_unwrap(env, obj, (void**)&a));
  a->n = n;
  a->dtype = dtype;
  if (like) {
    a->ndim = like->ndim;
    memcpy(a->shape, like->shape, sizeof a->shape);
  } else {
    a->ndim = 1;
    a->shape[0] = (int64_t)n;
  }
  if (n && hipMalloc(&a->data, n * (size_t)dtype_bytes(dtype)) != hipSuccess)
    return throw_code(env, "GenericFailure", "hipMalloc failed");
  *out = a;
  return obj;
}

static Array* unwrap_array(napi_env env, napi_value v) {
  napi_valuetype t;
  if (napi_typeof(env, v, &t) != napi_ok || t != napi_object) {
    throw_code(env, "InvalidArg", "expected an MxArray");
    return NULL;
  }
  napi_value ctor;
  bool is = false;
  if (napi_get_reference_value(env, g_array_ctor, &ctor) != napi_ok || napi_instanceof(env, v, ctor, &is) != napi_ok ||
      !is) {
    throw_code(env, "InvalidArg", "expected an MxArray");
    return NULL;
  }
  Array* a = NULL;
  if (napi_unwrap(env, v, (void**)&a) != napi_ok) return NULL;
  return a;
}

static mxopt_array as_c(const Array* a) {
  mxopt_array c = {a->data, a->n, a->dtype};
  return c;
}

/* shape: BigInt64Array (as the reference declares it) or a plain array of numbers */
static bool read_shape(napi_env env, napi_value v, Array* a) {
  bool is_typed = false;
  napi_is_typedarray(env, v, &is_typed);
  a->ndim = 0;
  a->n = 1;
  if (is_typed) {
    napi_typedarray_type type;
    size_t len;
    void* data;
    if (napi_get_typedarray_info(env, v, &type, &len, &data, NULL, NULL) != napi_ok || type != napi_bigint64_array || len > 8)
      return false;
    for (size_t i = 0; i < len; ++i) a->shape[a->ndim++] = ((int64_t*)data)[i];
  } else {
    uint32_t len = 0;
    if (napi_get_array_length(env, v, &len) != napi_ok || len > 8) return false;
    for (uint32_t i = 0; i < len; ++i) {
      napi_value e;
      double d;
      if (napi_get_element(env, v, i, &e) != napi_ok || napi_get_value_double(env, e, &d) != napi_ok) return false;
      a->shape[a->ndim++] = (int64_t)d;
    }
  }
  for (int i = 0; i < a->ndim; ++i) {
    if (a->shape[i] < 0) return false;
    a->n *= (uint64_t)a->shape[i];
  }
  return true;
}

static napi_value array_from_float32(napi_env env, napi_callback_info info) {
  size_t argc = 2;
  napi_value argv[2];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  if (argc < 2) return throw_code(env, "InvalidArg", "fromFloat32(data, shape)");
  napi_typedarray_type type;
  size_t len;
  void* data;
  if (napi_get_typedarray_info(env, argv[0], &type, &len, &data, NULL, NULL) != napi_ok || type != napi_float32_array)
    return throw_code(env, "InvalidArg", "fromFloat32: data must be a Float32Array");
  Array shape_only;
  if (!read_shape(env, argv[1], &shape_only)) return throw_code(env, "InvalidArg", "fromFloat32: bad shape");
  if (shape_only.n != len) return throw_code(env, "InvalidArg", "fromFloat32: data length does not match the shape");
  Array* a;
  napi_value obj = new_array(env, len, MXOPT_F32, &shape_only, &a);
  if (!obj) return NULL;
  if (len && hipMemcpy(a->data, data, len * 4, hipMemcpyHostToDevice) != hipSuccess)
    return throw_code(env, "GenericFailure", "hipMemcpy failed");
  return obj;
}

static napi_value array_zeros(napi_env env, napi_callback_info info) {
  size_t argc = 2;
  napi_value argv[2];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  Array shape_only;
  if (argc < 1 || !read_shape(env, argv[0], &shape_only)) return throw_code(env, "InvalidArg", "zeros: bad shape");
  int32_t dtype = MXOPT_F32;
  napi_valuetype t = napi_undefined;
  if (argc > 1) napi_typeof(env, argv[1], &t);
  if (t == napi_number) NAPI_OK(napi_get_value_int32(env, argv[1], &dtype));
  if (dtype != MXOPT_F32 && dtype != MXOPT_F16 && dtype != MXOPT_BF16)
    return throw_code(env, "InvalidArg", "zeros: only floating dtypes are supported here");
  Array* a;
  napi_value obj = new_array(env, shape_only.n, dtype, &shape_only, &a);
  if (!obj) return NULL;
  if (a->n && hipMemset(a->data, 0, a->n * (size_t)dtype_bytes(dtype)) != hipSuccess)
    return throw_code(env, "GenericFailure", "hipMemset failed");
  return obj;
}

static float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const int exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do { ++e; man <<= 1; } while (!(man & 0x400u));
      bits = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | man << 13;
  } else {
    bits = sign | (uint32_t)(exp - 15 + 127) << 23 | man << 13;
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static napi_value array_to_float32(napi_env env, napi_callback_info info) {
  napi_value self;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Array* a = unwrap_array(env, self);
  if (!a) return NULL;
  MX_OK(mxopt_synchronize(g_ctx));
  napi_value buffer, out;
  float* dst;
  NAPI_OK(napi_create_arraybuffer(env, a->n * 4, (void**)&dst, &buffer));
  if (a->n) {
    if (a->dtype == MXOPT_F32) {
      if (hipMemcpy(dst, a->data, a->n * 4, hipMemcpyDeviceToHost) != hipSuccess)
        return throw_code(env, "GenericFailure", "hipMemcpy failed");
    } else {
      uint16_t* tmp = (uint16_t*)malloc(a->n * 2);
      if (!tmp || hipMemcpy(tmp, a->data, a->n * 2, hipMemcpyDeviceToHost) != hipSuccess) {
        free(tmp);
        return throw_code(env, "GenericFailure", "hipMemcpy failed");
      }
      for (uint64_t i = 0; i < a->n; ++i) {
        if (a->dtype == MXOPT_BF16) {
          uint32_t bits = (uint32_t)tmp[i] << 16;
          memcpy(&dst[i], &bits, 4);
        } else {
          dst[i] = half_to_float(tmp[i]);
        }
      }
      free(tmp);
    }
  }
  NAPI_OK(napi_create_typedarray(env, napi_float32_array, a->n, buffer, 0, &out));
  return out;
}

static napi_value array_shape(napi_env env, napi_callback_info info) {
  napi_value self, buffer, out;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Array* a = unwrap_array(env, self);
  if (!a) return NULL;
  int64_t* dst;
  NAPI_OK(napi_create_arraybuffer(env, (size_t)a->ndim * 8, (void**)&dst, &buffer));
  memcpy(dst, a->shape, (size_t)a->ndim * 8);
  NAPI_OK(napi_create_typedarray(env, napi_bigint64_array, (size_t)a->ndim, buffer, 0, &out));
  return out;
}

static napi_value array_size(napi_env env, napi_callback_info info) {
  napi_value self, out;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Array* a = unwrap_array(env, self);
  if (!a) return NULL;
  NAPI_OK(napi_create_bigint_uint64(env, a->n, &out));
  return out;
}

static napi_value array_dtype(napi_env env, napi_callback_info info) {
  napi_value self, out;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Array* a = unwrap_array(env, self);
  if (!a) return NULL;
  NAPI_OK(napi_create_int32(env, a->dtype, &out));
  return out;
}

/* astype: the copy-with-conversion that a first accumulation is (round to nearest even) */
static napi_value array_astype(napi_env env, napi_callback_info info) {
  size_t argc = 1;
  napi_value argv[1], self;
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, &self, NULL));
  Array* a = unwrap_array(env, self);
  if (!a) return NULL;
  int32_t dtype;
  if (argc < 1 || napi_get_value_int32(env, argv[0], &dtype) != napi_ok) return throw_code(env, "InvalidArg", "astype(dtype)");
  if (dtype != MXOPT_F32 && dtype != MXOPT_F16 && dtype != MXOPT_BF16)
    return throw_code(env, "InvalidArg", "astype: only floating dtypes are supported here");
  Array* o;
  napi_value obj = new_array(env, a->n, dtype, a, &o);
  if (!obj) return NULL;
  const mxopt_array none = {NULL, 0, 0}, src = as_c(a), dst = as_c(o);
  MX_OK(mxopt_accumulate_gradients(g_ctx, 1, &none, &src, &dst));
  return obj;
}

/* ---- optimizers --------------------------------------------------------------------- */

static void optimizer_finalize(napi_env env, void* data, void* hint) {
  (void)env; (void)hint;
  Optimizer* o = (Optimizer*)data;
  if (o->opt) mxopt_optimizer_free(o->opt);
  free(o);
}

/* number | undefined | null -> pointer to the value or NULL */
static const double* opt_double(napi_env env, napi_value v, double* slot) {
  napi_valuetype t;
  if (napi_typeof(env, v, &t) != napi_ok || t != napi_number) return NULL;
  return napi_get_value_double(env, v, slot) == napi_ok ? slot : NULL;
}
static const int* opt_bool(napi_env env, napi_value v, int* slot) {
  napi_valuetype t;
  bool b;
  if (napi_typeof(env, v, &t) != napi_ok || t != napi_boolean || napi_get_value_bool(env, v, &b) != napi_ok) return NULL;
  *slot = b;
  return slot;
}

enum { KIND_ADAM, KIND_ADAMW, KIND_SGD, KIND_RMSPROP };

static napi_value optimizer_construct(napi_env env, napi_callback_info info) {
  size_t argc = 6;
  napi_value argv[6], self, undefined;
  void* kind_ptr;
  NAPI_OK(napi_get_undefined(env, &undefined));
  for (int i = 0; i < 6; ++i) argv[i] = undefined;
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, &self, &kind_ptr));
  const int kind = (int)(intptr_t)kind_ptr;
  double d[5];
  int b[1];
  Optimizer* o = (Optimizer*)calloc(1, sizeof *o);
  if (!o) return throw_code(env, "GenericFailure", "out of memory");
  int rc;
  switch (kind) {
    case KIND_ADAM:
      rc = mxopt_adam_new(g_ctx, opt_double(env, argv[0], &d[0]), opt_double(env, argv[1], &d[1]),
                          opt_double(env, argv[2], &d[2]), opt_double(env, argv[3], &d[3]), opt_bool(env, argv[4], &b[0]),
                          &o->opt);
      break;
    case KIND_ADAMW:
      rc = mxopt_adamw_new(g_ctx, opt_double(env, argv[0], &d[0]), opt_double(env, argv[1], &d[1]),
                           opt_double(env, argv[2], &d[2]), opt_double(env, argv[3], &d[3]),
                           opt_double(env, argv[4], &d[4]), opt_bool(env, argv[5], &b[0]), &o->opt);
      break;
    case KIND_SGD: {
      double lr;
      if (napi_get_value_double(env, argv[0], &lr) != napi_ok) {
        free(o);
        return throw_code(env, "InvalidArg", "SGD: learningRate is required");
      }
      rc = mxopt_sgd_new(g_ctx, lr, opt_double(env, argv[1], &d[1]), opt_double(env, argv[2], &d[2]),
                         opt_double(env, argv[3], &d[3]), opt_bool(env, argv[4], &b[0]), &o->opt);
      break;
    }
    default:
      rc = mxopt_rmsprop_new(g_ctx, opt_double(env, argv[0], &d[0]), opt_double(env, argv[1], &d[1]),
                             opt_double(env, argv[2], &d[2]), opt_double(env, argv[3], &d[3]), &o->opt);
  }
  if (rc != MXOPT_OK) {
    free(o);
    return throw_status(env, rc);
  }
  NAPI_OK(napi_wrap(env, self, o, optimizer_finalize, NULL, NULL));
  return self;
}

static napi_value optimizer_update_single(napi_env env, napi_callback_info info) {
  size_t argc = 3;
  napi_value argv[3], self;
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, &self, NULL));
  if (argc < 3) return throw_code(env, "InvalidArg", "updateSingle(paramName, param, grad)");
  Optimizer* o;
  NAPI_OK(napi_unwrap(env, self, (void**)&o));
  char name[512];
  size_t len;
  if (napi_get_value_string_utf8(env, argv[0], name, sizeof name, &len) != napi_ok)
    return throw_code(env, "InvalidArg", "updateSingle: paramName must be a string");
  Array *p = unwrap_array(env, argv[1]), *g = p ? unwrap_array(env, argv[2]) : NULL;
  if (!p || !g) return NULL;
  Array* out;
  /* float32, as the reference's op chain returns (adamw.rs:116: nothing casts back) */
  napi_value obj = new_array(env, p->n, MXOPT_F32, p, &out);
  if (!obj) return NULL;
  const mxopt_array ap = as_c(p), ag = as_c(g), ao = as_c(out);
  MX_OK(mxopt_optimizer_update_single(o->opt, name, &ap, &ag, &ao));
  return obj;
}

static napi_value optimizer_reset(napi_env env, napi_callback_info info) {
  napi_value self;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  Optimizer* o;
  NAPI_OK(napi_unwrap(env, self, (void**)&o));
  MX_OK(mxopt_optimizer_reset(o->opt));
  return NULL;
}

/* ---- Record<string, MxArray> helpers ---------------------------------------------------- */

typedef struct {
  uint32_t n;
  napi_value keys;
  mxopt_array* in;
  Array** arrays;
} Record;

static bool read_record(napi_env env, napi_value obj, Record* r) {
  memset(r, 0, sizeof *r);
  if (napi_get_property_names(env, obj, &r->keys) != napi_ok || napi_get_array_length(env, r->keys, &r->n) != napi_ok) {
    throw_code(env, "InvalidArg", "expected an object of MxArray values");
    return false;
  }
  r->in = (mxopt_array*)calloc(r->n ? r->n : 1, sizeof *r->in);
  r->arrays = (Array**)calloc(r->n ? r->n : 1, sizeof *r->arrays);
  for (uint32_t i = 0; i < r->n; ++i) {
    napi_value key, val;
    if (napi_get_element(env, r->keys, i, &key) != napi_ok || napi_get_property(env, obj, key, &val) != napi_ok ||
        !(r->arrays[i] = unwrap_array(env, val))) {
      free(r->in);
      free(r->arrays);
      return false;
    }
    r->in[i] = as_c(r->arrays[i]);
  }
  return true;
}

static void free_record(Record* r) {
  free(r->in);
  free(r->arrays);
}

/* A new object with the keys of `r` and freshly allocated arrays of `dtype(i)`. */
static napi_value new_record_like(napi_env env, const Record* r, const int* dtypes, mxopt_array* outs) {
  napi_value obj;
  NAPI_OK(napi_create_object(env, &obj));
  for (uint32_t i = 0; i < r->n; ++i) {
    napi_value key;
    Array* o;
    NAPI_OK(napi_get_element(env, r->keys, i, &key));
    napi_value arr = new_array(env, r->arrays[i]->n, dtypes ? dtypes[i] : MXOPT_F32, r->arrays[i], &o);
    if (!arr) return NULL;
    outs[i] = as_c(o);
    NAPI_OK(napi_set_property(env, obj, key, arr));
  }
  return obj;
}

/* ---- GradientUtils ---------------------------------------------------------------------- */

static napi_value gu_compute_gradient_norm(napi_env env, napi_callback_info info) {
  size_t argc = 1;
  napi_value argv[1], out;
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  Record r;
  if (argc < 1 || !read_record(env, argv[0], &r)) return NULL;
  double norm = 0.0;
  int rc = mxopt_compute_gradient_norm(g_ctx, r.n, r.in, &norm);
  free_record(&r);
  if (rc) return throw_status(env, rc);
  NAPI_OK(napi_create_double(env, norm, &out));
  return out;
}

static napi_value clip_norm_common(napi_env env, napi_callback_info info, bool with_norm) {
  size_t argc = 2;
  napi_value argv[2];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  double max_norm;
  if (argc < 2 || napi_get_value_double(env, argv[1], &max_norm) != napi_ok)
    return throw_code(env, "InvalidArg", "clipGradNorm(gradients, maxNorm)");
  Record r;
  if (!read_record(env, argv[0], &r)) return NULL;
  mxopt_array* outs = (mxopt_array*)calloc(r.n ? r.n : 1, sizeof *outs);
  napi_value obj = new_record_like(env, &r, NULL, outs);
  double norm = 0.0;
  int rc = obj ? mxopt_clip_grad_norm(g_ctx, r.n, r.in, max_norm, outs, with_norm ? &norm : NULL) : MXOPT_OK;
  free(outs);
  free_record(&r);
  if (!obj) return NULL;
  if (rc) return throw_status(env, rc);
  if (!with_norm) return obj;
  napi_value pair, n;
  NAPI_OK(napi_create_array_with_length(env, 2, &pair));
  NAPI_OK(napi_create_double(env, norm, &n));
  NAPI_OK(napi_set_element(env, pair, 0, obj));
  NAPI_OK(napi_set_element(env, pair, 1, n));
  return pair;
}
static napi_value gu_clip_grad_norm(napi_env env, napi_callback_info info) { return clip_norm_common(env, info, false); }
static napi_value gu_clip_grad_norm_with_norm(napi_env env, napi_callback_info info) {
  return clip_norm_common(env, info, true);
}

static napi_value gu_clip_grad_value(napi_env env, napi_callback_info info) {
  size_t argc = 3;
  napi_value argv[3];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  double lo, hi;
  if (argc < 3 || napi_get_value_double(env, argv[1], &lo) != napi_ok || napi_get_value_double(env, argv[2], &hi) != napi_ok)
    return throw_code(env, "InvalidArg", "clipGradValue(grad, minVal, maxVal)");
  Array* g = unwrap_array(env, argv[0]);
  if (!g) return NULL;
  Array* o;
  napi_value obj = new_array(env, g->n, MXOPT_F32, g, &o);
  if (!obj) return NULL;
  const mxopt_array ag = as_c(g), ao = as_c(o);
  MX_OK(mxopt_clip_grad_value(g_ctx, &ag, lo, hi, &ao));
  return obj;
}

/* ---- clipGradientsByGlobalNorm / clipGradientsByValue (Array<MxArray>) ---------------------- */

static napi_value clip_list_common(napi_env env, napi_callback_info info, bool by_value) {
  size_t argc = 3;
  napi_value argv[3];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  double a = 0, b = 0;
  if (argc < (by_value ? 3u : 2u) || napi_get_value_double(env, argv[1], &a) != napi_ok ||
      (by_value && napi_get_value_double(env, argv[2], &b) != napi_ok))
    return throw_code(env, "InvalidArg", "expected (gradients, bound[, bound])");
  uint32_t n = 0;
  NAPI_OK(napi_get_array_length(env, argv[0], &n));
  mxopt_array* in = (mxopt_array*)calloc(n ? n : 1, sizeof *in);
  mxopt_array* outs = (mxopt_array*)calloc(n ? n : 1, sizeof *outs);
  napi_value list;
  NAPI_OK(napi_create_array_with_length(env, n, &list));
  for (uint32_t i = 0; i < n; ++i) {
    napi_value e;
    Array *g, *o;
    if (napi_get_element(env, argv[0], i, &e) != napi_ok || !(g = unwrap_array(env, e))) { free(in); free(outs); return NULL; }
    napi_value arr = new_array(env, g->n, MXOPT_F32, g, &o);
    if (!arr) { free(in); free(outs); return NULL; }
    in[i] = as_c(g);
    outs[i] = as_c(o);
    NAPI_OK(napi_set_element(env, list, i, arr));
  }
  int rc = by_value ? mxopt_clip_gradients_by_value(g_ctx, n, in, a, b, outs)
                    : mxopt_clip_gradients_by_global_norm(g_ctx, n, in, a, outs);
  free(in);
  free(outs);
  if (rc) return throw_status(env, rc);
  return list;
}
static napi_value clip_gradients_by_global_norm(napi_env env, napi_callback_info info) {
  return clip_list_common(env, info, false);
}
static napi_value clip_gradients_by_value(napi_env env, napi_callback_info info) {
  return clip_list_common(env, info, true);
}

/* ---- Qwen3Model.accumulateGradients (static) ------------------------------------------------ */

static napi_value accumulate_gradients(napi_env env, napi_callback_info info) {
  size_t argc = 2;
  napi_value argv[2];
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  if (argc < 2) return throw_code(env, "InvalidArg", "accumulateGradients(accumulatedGradients, newGradients)");
  Record fresh;
  if (!read_record(env, argv[1], &fresh)) return NULL;
  mxopt_array* acc = (mxopt_array*)calloc(fresh.n ? fresh.n : 1, sizeof *acc);
  mxopt_array* outs = (mxopt_array*)calloc(fresh.n ? fresh.n : 1, sizeof *outs);
  int* dtypes = (int*)calloc(fresh.n ? fresh.n : 1, sizeof *dtypes);
  napi_value result = NULL;
  int rc = MXOPT_OK;
  bool ok = true;
  for (uint32_t i = 0; i < fresh.n && ok; ++i) {   /* dtype = promote(acc, new) (model.rs:2227) */
    napi_value key, val;
    bool has = false;
    ok = napi_get_element(env, fresh.keys, i, &key) == napi_ok && napi_has_property(env, argv[0], key, &has) == napi_ok;
    dtypes[i] = fresh.arrays[i]->dtype;
    if (ok && has) {
      Array* a;
      ok = napi_get_property(env, argv[0], key, &val) == napi_ok && (a = unwrap_array(env, val)) != NULL;
      if (ok) {
        acc[i] = as_c(a);
        if (a->dtype != dtypes[i]) dtypes[i] = MXOPT_F32;
        if (a->dtype != dtypes[i]) {
          throw_code(env, "InvalidArg", "accumulateGradients: a 16-bit accumulator cannot take a float32 gradient");
          ok = false;
        }
      }
    }
  }
  if (ok) result = new_record_like(env, &fresh, dtypes, outs);
  if (ok && result) rc = mxopt_accumulate_gradients(g_ctx, fresh.n, acc, fresh.in, outs);
  /* names only in the accumulator are carried over (model.rs:2235-2240) */
  if (ok && result && rc == MXOPT_OK) {
    Record old;
    if (read_record(env, argv[0], &old)) {
      for (uint32_t i = 0; i < old.n && ok; ++i) {
        napi_value key, val;
        bool has = false;
        ok = napi_get_element(env, old.keys, i, &key) == napi_ok && napi_has_property(env, argv[1], key, &has) == napi_ok;
        if (ok && !has) ok = napi_get_property(env, argv[0], key, &val) == napi_ok &&
                             napi_set_property(env, result, key, val) == napi_ok;
      }
      free_record(&old);
    } else {
      ok = false;
    }
  }
  free(acc); free(outs); free(dtypes);
  free_record(&fresh);
  if (rc) return throw_status(env, rc);
  return ok ? result : NULL;
}

/* ---- LRScheduler ------------------------------------------------------------------------- */

static napi_value lr_common(napi_env env, napi_callback_info info, int which) {
  size_t argc = 4;
  napi_value argv[4], out;
  NAPI_OK(napi_get_cb_info(env, info, &argc, argv, NULL, NULL));
  double a, b, c, d;
  if (argc < 4 || napi_get_value_double(env, argv[0], &a) != napi_ok || napi_get_value_double(env, argv[1], &b) != napi_ok ||
      napi_get_value_double(env, argv[2], &c) != napi_ok || napi_get_value_double(env, argv[3], &d) != napi_ok)
    return throw_code(env, "InvalidArg", "expected four numbers");
  double v;
  switch (which) {
    case 0: v = mxopt_lr_linear_decay(a, b, (int64_t)c, (int64_t)d); break;
    case 1: v = mxopt_lr_exponential_decay(a, b, (int64_t)c, (int64_t)d); break;
    case 2: v = mxopt_lr_cosine_annealing(a, b, (int64_t)c, (int64_t)d); break;
    default: v = mxopt_lr_step_decay(a, b, (int64_t)c, (int64_t)d);
  }
  NAPI_OK(napi_create_double(env, v, &out));
  return out;
}
static napi_value lr_linear(napi_env e, napi_callback_info i) { return lr_common(e, i, 0); }
static napi_value lr_exponential(napi_env e, napi_callback_info i) { return lr_common(e, i, 1); }
static napi_value lr_cosine(napi_env e, napi_callback_info i) { return lr_common(e, i, 2); }
static napi_value lr_step(napi_env e, napi_callback_info i) { return lr_common(e, i, 3); }

/* ---- module ------------------------------------------------------------------------------- */

#define METHOD(name, fn) {name, NULL, fn, NULL, NULL, NULL, napi_default, NULL}
#define STATIC(name, fn) {name, NULL, fn, NULL, NULL, NULL, napi_static, NULL}

static napi_value noop_construct(napi_env env, napi_callback_info info) {
  napi_value self;
  NAPI_OK(napi_get_cb_info(env, info, NULL, NULL, &self, NULL));
  return self;
}

static napi_value init(napi_env env, napi_value exports) {
  if (mxopt_create(0, NULL, &g_ctx) != MXOPT_OK) return throw_code(env, "GenericFailure", mxopt_last_error(NULL));

  const napi_property_descriptor array_props[] = {
      STATIC("fromFloat32", array_from_float32), STATIC("zeros", array_zeros), METHOD("toFloat32", array_to_float32),
      METHOD("shape", array_shape), METHOD("size", array_size), METHOD("dtype", array_dtype), METHOD("astype", array_astype)};
  napi_value array_class;
  NAPI_OK(napi_define_class(env, "MxArray", NAPI_AUTO_LENGTH, array_construct, NULL,
                            sizeof array_props / sizeof *array_props, array_props, &array_class));
  NAPI_OK(napi_create_reference(env, array_class, 1, &g_array_ctor));
  NAPI_OK(napi_set_named_property(env, exports, "MxArray", array_class));

  const napi_property_descriptor opt_props[] = {METHOD("updateSingle", optimizer_update_single),
                                                METHOD("reset", optimizer_reset)};
  const char* names[] = {"Adam", "AdamW", "SGD", "RMSprop"};
  for (int k = 0; k < 4; ++k) {
    napi_value cls;
    NAPI_OK(napi_define_class(env, names[k], NAPI_AUTO_LENGTH, optimizer_construct, (void*)(intptr_t)k, 2, opt_props, &cls));
    NAPI_OK(napi_set_named_property(env, exports, names[k], cls));
  }

  const napi_property_descriptor gu_props[] = {
      STATIC("computeGradientNorm", gu_compute_gradient_norm), STATIC("clipGradNorm", gu_clip_grad_norm),
      STATIC("clipGradNormWithNorm", gu_clip_grad_norm_with_norm), STATIC("clipGradValue", gu_clip_grad_value)};
  napi_value gu;
  NAPI_OK(napi_define_class(env, "GradientUtils", NAPI_AUTO_LENGTH, noop_construct, NULL, 4, gu_props, &gu));
  NAPI_OK(napi_set_named_property(env, exports, "GradientUtils", gu));

  const napi_property_descriptor lr_props[] = {STATIC("linearDecay", lr_linear), STATIC("exponentialDecay", lr_exponential),
                                               STATIC("cosineAnnealing", lr_cosine), STATIC("stepDecay", lr_step)};
  napi_value lr;
  NAPI_OK(napi_define_class(env, "LRScheduler", NAPI_AUTO_LENGTH, noop_construct, NULL, 4, lr_props, &lr));
  NAPI_OK(napi_set_named_property(env, exports, "LRScheduler", lr));

  const napi_property_descriptor model_props[] = {STATIC("accumulateGradients", accumulate_gradients)};
  napi_value model;
  NAPI_OK(napi_define_class(env, "Qwen3Model", NAPI_AUTO_LENGTH, noop_construct, NULL, 1, model_props, &model));
  NAPI_OK(napi_set_named_property(env, exports, "Qwen3Model", model));

  napi_value fn;
  NAPI_OK(napi_create_function(env, "clipGradientsByGlobalNorm", NAPI_AUTO_LENGTH, clip_gradients_by_global_norm, NULL, &fn));
  NAPI_OK(napi_set_named_property(env, exports, "clipGradientsByGlobalNorm", fn));
  NAPI_OK(napi_create_function(env, "clipGradientsByValue", NAPI_AUTO_LENGTH, clip_gradients_by_value, NULL, &fn));
  NAPI_OK(napi_set_named_property(env, exports, "clipGradientsByValue", fn));

  napi_value dtype, v;
  NAPI_OK(napi_create_object(env, &dtype));
  const char* dnames[] = {"Float32", "Int32", "Float16", "BFloat16", "Uint32"};
  for (int i = 0; i < 5; ++i) {
    NAPI_OK(napi_create_int32(env, i, &v));
    NAPI_OK(napi_set_named_property(env, dtype, dnames[i], v));
  }
  NAPI_OK(napi_set_named_property(env, exports, "DType", dtype));
  return exports;
}

NAPI_MODULE(mxopt, init)
