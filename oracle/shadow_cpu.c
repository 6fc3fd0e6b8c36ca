/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement, in plain C, of the loops that junluan/shadow runs on the host
 * for its Unary / Binary / Eltwise / Reduce / Activate / Scale operators, and for
 * the operators next to them (Axpy, BatchNorm, LRN, GridSample, Pooling, Softmax,
 * Normalize, SSDNormalize, Group/Instance/LayerNorm, and the data movers), when
 * built without Eigen/BLAS/DNNL (the "plain loop + libm" branch).  It is the
 * checker for the HIP kernels and the CPU leg of the benchmark; nothing under
 * shadow_amd/ may call it.
 *
 * Every function names the reference lines it follows.  Built with the
 * reference's Release flags (-O3 -DNDEBUG, no -march, no fast-math) plus
 * -ffp-contract=off.  Transcendentals are the host's libm, as in the reference.
 *
 * Pinning (see tests/test_oracle_*.py): IEEE closed forms against numpy fp32,
 * brute-force N-d broadcast and reduce written independently in numpy, exact
 * integer-valued sums, signed-zero / NaN special cases, libm results against
 * fp64 evaluations within 1 ulp.  The reference holds no test vectors for this
 * path and its own build needs a cmake-generated header, so no compiled
 * reference backs these checks.
 *
 * Parity unpinned: the last bit of everything that comes from libm (orc_unary's
 * log / exp / sin / cos / tan / asin / acos / atan, pow, sigmoid, softplus, tanh,
 * gelu, the expf inside softmax, the powf inside normalize and lrn) is whatever the
 * host's libm gives, as in the reference; tests/golden/libm_glibc235.npz records
 * the glibc 2.35 values the device code is built to.  orc_grid_sample: a coordinate
 * that fits no int, and a NaN coordinate in the bilinear mode (see there).
 */
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define API __attribute__((visibility("default")))

/* std::max / std::min as libstdc++ defines them */
static inline float std_max(float a, float b) { return (a < b) ? b : a; }
static inline float std_min(float a, float b) { return (b < a) ? b : a; }

/* ---- shadow/core/blas.cpp:25-34  Blas::Set ---- */
API void orc_set(int n, float val, float* y) {
  for (int i = 0; i < n; ++i) y[i] = val;
}

/* ---- shadow/core/blas.cpp:143-168  15 unary ops (loop branch);
 *      enum values shadow/operators/kernels/unary.hpp:9-25 ---- */
API int orc_unary(int op, int n, const float* a, float* y) {
  switch (op) {
    case 0: for (int i = 0; i < n; ++i) y[i] = fabsf(a[i]); break;
    case 1: for (int i = 0; i < n; ++i) y[i] = a[i] * a[i]; break;
    case 2: for (int i = 0; i < n; ++i) y[i] = sqrtf(a[i]); break;
    case 3: for (int i = 0; i < n; ++i) y[i] = logf(a[i]); break;
    case 4: for (int i = 0; i < n; ++i) y[i] = expf(a[i]); break;
    case 5: for (int i = 0; i < n; ++i) y[i] = sinf(a[i]); break;
    case 6: for (int i = 0; i < n; ++i) y[i] = cosf(a[i]); break;
    case 7: for (int i = 0; i < n; ++i) y[i] = tanf(a[i]); break;
    case 8: for (int i = 0; i < n; ++i) y[i] = asinf(a[i]); break;
    case 9: for (int i = 0; i < n; ++i) y[i] = acosf(a[i]); break;
    case 10: for (int i = 0; i < n; ++i) y[i] = atanf(a[i]); break;
    case 11: for (int i = 0; i < n; ++i) y[i] = floorf(a[i]); break;
    case 12: for (int i = 0; i < n; ++i) y[i] = ceilf(a[i]); break;
    case 13: for (int i = 0; i < n; ++i) y[i] = -a[i]; break;
    case 14: for (int i = 0; i < n; ++i) y[i] = 1 / a[i]; break;
    default: return -1;
  }
  return 0;
}

/* one binary op on two values: shadow/core/blas.cpp:114-120 and
 * shadow/operators/kernels/binary.cpp:9-28; enum binary.hpp:23 */
static inline float binary_one(float a, float b, int op) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 3: return a / b;
    case 4: return powf(a, b);
    case 5: return std_max(a, b);
    case 6: return std_min(a, b);
    default: return 0;
  }
}

/* ---- shadow/core/blas.cpp:103-121  tensor (op) tensor ---- */
API int orc_binary(int op, int n, const float* a, const float* b, float* y) {
  if (op < 0 || op > 6) return -1;
  for (int i = 0; i < n; ++i) y[i] = binary_one(a[i], b[i], op);
  return 0;
}

/* ---- shadow/core/blas.cpp:123-141  tensor (op) scalar ---- */
API int orc_binary_scalar(int op, int n, const float* a, float alpha, float* y) {
  if (op < 0 || op > 6) return -1;
  for (int i = 0; i < n; ++i) y[i] = binary_one(a[i], alpha, op);
  return 0;
}

/* ---- shadow/core/blas.cpp:172-235  level 1 (loop branch) ---- */
API void orc_scal(int n, float alpha, float* x) {
  for (int i = 0; i < n; ++i) x[i] *= alpha;
}
API void orc_copy(int n, const float* x, float* y) {
  for (int i = 0; i < n; ++i) y[i] = x[i];
}
API void orc_axpy(int n, float alpha, const float* x, float* y) {
  for (int i = 0; i < n; ++i) y[i] += alpha * x[i];
}
API float orc_asum(int n, const float* x) {
  double asum = 0;
  for (int i = 0; i < n; ++i) asum += fabsf(x[i]);
  return (float)asum;
}

/* ---- shadow/operators/kernels/binary.cpp:30-52  Vision::BroadcastBinary ----
 * shapes are rank-aligned; broadcasting is the "% shape" on each operand. */
API int orc_broadcast_binary(const float* in, const int* in_shape, const float* sc,
                             const int* sc_shape, int op, int num_axes, int count,
                             const int* out_shape, float* out) {
  if (op < 0 || op > 6 || num_axes < 1) return -1;
  int* in_acc = (int*)malloc(sizeof(int) * num_axes);
  int* sc_acc = (int*)malloc(sizeof(int) * num_axes);
  in_acc[num_axes - 1] = 1;
  sc_acc[num_axes - 1] = 1;
  for (int n = num_axes - 1; n > 0; --n) {
    in_acc[n - 1] = in_shape[n] * in_acc[n];
    sc_acc[n - 1] = sc_shape[n] * sc_acc[n];
  }
  for (int i = 0; i < count; ++i) {
    int in_index = 0, sc_index = 0, cc = i;
    for (int n = num_axes - 1; n >= 0; --n) {
      int dim = cc % out_shape[n];
      in_index += (dim % in_shape[n]) * in_acc[n];
      sc_index += (dim % sc_shape[n]) * sc_acc[n];
      cc /= out_shape[n];
    }
    out[i] = binary_one(in[in_index], sc[sc_index], op);
  }
  free(in_acc);
  free(sc_acc);
  return 0;
}

/* ---- shadow/operators/kernels/activate.cpp:9-39  Vision::Activate ----
 * enum shadow/operators/kernels/activate.hpp:24-34 (0 = PRelu, see below) */
static inline float activate_one(float x, int type, float slope) {
  switch (type) {
    case 1: return x > 0 ? x : 0;
    case 2: return x > 0 ? x : slope * x;
    case 3: return 1 / (1 + expf(-x));
    case 4: return log1pf(expf(x));
    case 5: return tanhf(x);
    case 6: return x < 0 ? 0 : (x > 6 ? 6 : x);
    case 7: return x < -3 ? 0 : (x > 3 ? x : (x * (x + 3) / 6.f));
    case 8: return 0.5f * x * (1 + erff(0.707107f * x));
    default: return x;
  }
}
API void orc_activate(const float* in, float* out, int count, int type, float slope) {
  for (int i = 0; i < count; ++i) out[i] = activate_one(in[i], type, slope);
}

/* ---- shadow/operators/kernels/activate.cpp:41-53  Vision::PRelu ---- */
API void orc_prelu(const float* in, float* out, const int* in_shape, int num_axes,
                   int channel_shared, const float* slope) {
  int channels = in_shape[1], dim = 1;
  for (int i = 2; i < num_axes; ++i) dim *= in_shape[i];
  int count = in_shape[0] * channels * dim;
  int div_factor = channel_shared ? channels : 1;
  for (int i = 0; i < count; ++i) {
    int c = (i / dim) % channels / div_factor;
    out[i] = in[i] > 0 ? in[i] : in[i] * slope[c];
  }
}

/* ---- shadow/operators/kernels/scale.cpp:7-39 ---- */
API void orc_scale_bias(const float* in, int count, const float* scale, const float* bias,
                        int scale_num, int inner_num, float* out) {
  for (int i = 0; i < count; ++i) {
    int index = (i / inner_num) % scale_num;
    out[i] = in[i] * scale[index] + bias[index];
  }
}
API void orc_scale(const float* in, int count, const float* scale, int scale_num,
                   int inner_num, float* out) {
  for (int i = 0; i < count; ++i) {
    int index = (i / inner_num) % scale_num;
    out[i] = in[i] * scale[index];
  }
}
API void orc_bias(const float* in, int count, const float* bias, int scale_num, int inner_num,
                  float* out) {
  for (int i = 0; i < count; ++i) {
    int index = (i / inner_num) % scale_num;
    out[i] = in[i] + bias[index];
  }
}

/* ---- shadow/operators/kernels/eltwise.hpp:18-71  EltwiseKernelDefault::Run ----
 * enum eltwise.hpp:9: 0 Prod, 1 Sum, 2 Max, 3 Min.  Written as the same chain
 * of whole-array passes, so aliasing out with an input behaves as it does there. */
API int orc_eltwise(int op, int k, const float* const* in, const float* coeff, int count,
                    float* out) {
  if (k < 2) return -1;
  switch (op) {
    case 0:
      orc_binary(2, count, in[0], in[1], out);
      for (int n = 2; n < k; ++n) orc_binary(2, count, out, in[n], out);
      break;
    case 1:
      orc_set(count, 0, out);
      for (int n = 0; n < k; ++n) orc_axpy(count, coeff[n], in[n], out);
      break;
    case 2:
      orc_binary(5, count, in[0], in[1], out);
      for (int n = 2; n < k; ++n) orc_binary(5, count, out, in[n], out);
      break;
    case 3:
      orc_binary(6, count, in[0], in[1], out);
      for (int n = 2; n < k; ++n) orc_binary(6, count, out, in[n], out);
      break;
    default:
      return -1;
  }
  return 0;
}

/* ---- shadow/operators/kernels/reduce.cpp:9-65  inline Reduce() ---- */
static float reduce_one(const float* data, const int* list, int num_list, int offset, int op) {
  switch (op) {
    case 0: {
      double val = 1;
      for (int i = 0; i < num_list; ++i) val *= data[list[i] + offset];
      return (float)val;
    }
    case 1: {
      double val = 0;
      for (int i = 0; i < num_list; ++i) val += data[list[i] + offset];
      return (float)val;
    }
    case 2: {
      float val = -FLT_MAX; /* numeric_limits<float>::lowest() */
      for (int i = 0; i < num_list; ++i) val = std_max(val, data[list[i] + offset]);
      return val;
    }
    case 3: {
      float val = FLT_MAX;
      for (int i = 0; i < num_list; ++i) val = std_min(val, data[list[i] + offset]);
      return val;
    }
    case 4: {
      double val = 0;
      for (int i = 0; i < num_list; ++i) val += data[list[i] + offset];
      return (float)(val / num_list);
    }
    case 5: {
      double val = 0;
      for (int i = 0; i < num_list; ++i) val += fabsf(data[list[i] + offset]);
      return (float)val;
    }
    case 6: {
      double val = 0;
      for (int i = 0; i < num_list; ++i) {
        float abs_data = fabsf(data[list[i] + offset]);
        val += abs_data * abs_data; /* fp32 product, widened afterwards */
      }
      return sqrtf((float)val);
    }
    default:
      return 0;
  }
}

/* ---- shadow/operators/kernels/reduce.hpp:41-71  the index lists of ReduceKernelDefault::Run:
 *      list[num_list] = offsets inside one window, last listed axis fastest;
 *      offset[out_count] = origin of every output.  The reference rebuilds them only
 *      when the input shape changes (reduce.hpp:45).  Returns num_list, or -1.
 *      out_shape = in_shape with the reduced axes set to 1 (reduce_op.cpp:38-42). */
API int orc_reduce_lists(const int* in_shape, int num_axes, const int* axes, int num_reduce, int* list,
                         int* offset) {
  int shape_acc[16], out_shape[16];
  if (num_axes > 16) return -1;
  if (num_axes > 0) shape_acc[num_axes - 1] = 1;
  for (int n = num_axes - 1; n > 0; --n) shape_acc[n - 1] = in_shape[n] * shape_acc[n];
  int out_count = 1;
  for (int n = 0; n < num_axes; ++n) out_shape[n] = in_shape[n];
  for (int k = 0; k < num_reduce; ++k) out_shape[axes[k]] = 1;
  for (int n = 0; n < num_axes; ++n) out_count *= out_shape[n];
  int num_list = 1;
  list[0] = 0;
  for (int n = num_reduce - 1; n >= 0; --n) {
    int axis = axes[n], cur = num_list;
    for (int k = 1; k < in_shape[axis]; ++k)
      for (int j = 0; j < cur; ++j) list[num_list++] = list[j] + k * shape_acc[axis];
  }
  for (int i = 0; i < out_count; ++i) {
    int off = 0, cc = i;
    for (int n = num_axes - 1; n >= 0; --n) {
      int dim = out_shape[n];
      off += (cc % dim) * shape_acc[n];
      cc /= dim;
    }
    offset[i] = off;
  }
  return num_list;
}

/* ---- shadow/operators/kernels/reduce.cpp:67-76  Vision::Reduce ---- */
API void orc_vision_reduce(const float* in, const int* list, const int* offset, int num_list, int operation,
                           int count, float* out) {
  for (int i = 0; i < count; ++i) out[i] = reduce_one(in, list, num_list, offset[i], operation);
}

/* ---- shadow/operators/kernels/reduce.hpp:41-88  both steps for one call ---- */
API int orc_reduce(int op, const float* in, const int* in_shape, int num_axes, const int* axes,
                   int num_reduce, float* out) {
  if (op < 0 || op > 6 || num_axes > 16) return -1;
  size_t cap = 1, out_count = 1;
  for (int k = 0; k < num_reduce; ++k) cap *= (size_t)in_shape[axes[k]];
  for (int n = 0; n < num_axes; ++n) out_count *= (size_t)in_shape[n];
  out_count /= cap;
  int* list = (int*)malloc(sizeof(int) * cap);
  int* offset = (int*)malloc(sizeof(int) * out_count);
  int num_list = orc_reduce_lists(in_shape, num_axes, axes, num_reduce, list, offset);
  orc_vision_reduce(in, list, offset, num_list, op, (int)out_count, out);
  free(list);
  free(offset);
  return 0;
}

/* ======================================================================
 * Operators next to the hot path (callers of the same Blas / Vision layer).
 * ====================================================================== */

/* ---- shadow/operators/kernels/axpy.cpp:9-21  Vision::Axpy: out = y, then one
 *      BlasSaxpy (shadow/core/blas.cpp:214-216) per row of inner_num ---- */
API void orc_axpy_rows(const float* alpha, const float* x, const float* y, int outer_num,
                       int inner_num, float* out) {
  memmove(out, y, (size_t)outer_num * inner_num * sizeof(float));
  for (int n = 0; n < outer_num; ++n) {
    int off = n * inner_num;
    for (int i = 0; i < inner_num; ++i) out[off + i] += alpha[n] * x[off + i];
  }
}

/* ---- shadow/operators/kernels/batch_norm.cpp:11-24  Vision::BatchNorm ---- */
API void orc_batch_norm(const float* in, int count, const float* mean, const float* variance,
                        int channel, int inner_num, float scale_factor, float eps, float* out) {
  for (int i = 0; i < count; ++i) {
    int index = (i / inner_num) % channel;
    out[i] = (in[i] - mean[index] * scale_factor) /
             sqrtf(fabsf(variance[index] * scale_factor) + eps);
  }
}

/* ---- shadow/operators/kernels/softmax.cpp:10-42  Vision::Softmax: four passes,
 *      std::max(x, running) for the maximum, fp32 running sum over dim ---- */
API void orc_softmax(const float* in, int outer_num, int dim, int inner_num, float* val,
                     float* out) {
  int val_count = outer_num * inner_num, count = val_count * dim;
  for (int i = 0; i < val_count; ++i) {
    int n = i / inner_num, s = i % inner_num;
    const float* p = in + n * dim * inner_num + s;
    float max_val = -FLT_MAX;
    for (int c = 0; c < dim; ++c, p += inner_num) max_val = std_max(*p, max_val);
    val[i] = max_val;
  }
  for (int i = 0; i < count; ++i) {
    int n = i / dim / inner_num, s = i % inner_num;
    out[i] = expf(in[i] - val[n * inner_num + s]);
  }
  for (int i = 0; i < val_count; ++i) {
    int n = i / inner_num, s = i % inner_num;
    const float* p = out + n * dim * inner_num + s;
    float sum = 0.f;
    for (int c = 0; c < dim; ++c, p += inner_num) sum += *p;
    val[i] = sum;
  }
  for (int i = 0; i < count; ++i) {
    int n = i / dim / inner_num, s = i % inner_num;
    out[i] /= val[n * inner_num + s];
  }
}

/* ---- shadow/operators/kernels/normalize.cpp:10-43  Vision::Normalize: fp64
 *      running sum over dim, then x / max(norm, eps) ---- */
API void orc_normalize(const float* in, int outer_num, int dim, int inner_num, float* val,
                       float p, float eps, float* out) {
  int val_count = outer_num * inner_num, count = val_count * dim;
  for (int i = 0; i < val_count; ++i) {
    int n = i / inner_num, s = i % inner_num;
    const float* q = in + n * dim * inner_num + s;
    double acc = 0;
    if (p == 1) {
      for (int c = 0; c < dim; ++c, q += inner_num) acc += fabsf(*q);
      val[i] = (float)acc;
    } else if (p == 2) {
      for (int c = 0; c < dim; ++c, q += inner_num) {
        float abs_data = fabsf(*q);
        acc += abs_data * abs_data; /* fp32 product, widened afterwards */
      }
      val[i] = sqrtf((float)acc);
    } else {
      /* std::pow(float, float) is the fp32 overload */
      for (int c = 0; c < dim; ++c, q += inner_num) acc += powf(fabsf(*q), p);
      val[i] = powf((float)acc, 1.f / p);
    }
  }
  for (int i = 0; i < count; ++i) {
    int n = i / dim / inner_num, s = i % inner_num;
    out[i] = in[i] / std_max(val[n * inner_num + s], eps);
  }
}

/* ---- shadow/operators/kernels/ssd_normalize.cpp:7-29  Vision::SSDNormalize: `out`
 *      holds the squares on entry; fp64 running sum over the channels, fp64
 *      square root, then in / val ---- */
API void orc_ssd_normalize(const float* in, int outer_num, int channels, int inner_num, float eps,
                           float* val, float* out) {
  int val_count = outer_num * inner_num, count = val_count * channels;
  for (int i = 0; i < val_count; ++i) {
    int n = i / inner_num, s = i % inner_num;
    const float* q = out + n * channels * inner_num + s;
    double sum = 0;
    for (int c = 0; c < channels; ++c, q += inner_num) sum += *q;
    val[i] = (float)sqrt(sum + eps);
  }
  for (int i = 0; i < count; ++i) {
    int n = i / channels / inner_num, s = i % inner_num;
    out[i] = in[i] / val[n * inner_num + s];
  }
}

/* ---- shadow/operators/kernels/ssd_normalize.hpp:36-83
 *      SSDNormalizeKernelDefault::Run: Square into the output, then per item
 *      Sasum and Mul by 1 / sqrt(sum + eps) (all fp32 after the sum) or the
 *      per-position form above; then Sscal by the shared scale or Scale by the
 *      per-channel one.  scale may be NULL.  val: batch * spatial_dim floats. ---- */
API void orc_ssd_normalize_run(const float* in, int batch, int channel, int spatial_dim,
                               int across_spatial, int channel_shared, float eps,
                               const float* scale, float* val, float* out) {
  int num = channel * spatial_dim, count = batch * num;
  orc_unary(1, count, in, out); /* Square */
  if (across_spatial) {
    for (int b = 0; b < batch; ++b) {
      int offset = b * num;
      float sum = orc_asum(num, out + offset);
      orc_binary_scalar(2, num, in + offset, 1.f / sqrtf(sum + eps), out + offset); /* Mul */
    }
  } else {
    orc_ssd_normalize(in, batch, channel, spatial_dim, eps, val, out);
  }
  if (scale) {
    if (channel_shared)
      orc_scal(count, scale[0], out);
    else
      orc_scale(out, count, scale, channel, spatial_dim, out);
  }
}

/* ---- shadow/operators/kernels/pooling.cpp:7-42  Vision::Pooling2D.
 *      pool_type 0 = max, 1 = average over the window clipped to input + pad ---- */
API void orc_pooling2d(const float* in, const int* in_shape, int pool_type, int kernel_h,
                       int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
                       const int* out_shape, float* out) {
  int batch = in_shape[0], channel = in_shape[1];
  int in_h = in_shape[2], in_w = in_shape[3];
  int out_h = out_shape[2], out_w = out_shape[3];
  for (int b = 0; b < batch; ++b) {
    for (int c = 0; c < channel; ++c, in += in_h * in_w) {
      for (int h = 0; h < out_h; ++h) {
        for (int w = 0; w < out_w; ++w) {
          int hstart = h * stride_h - pad_h, wstart = w * stride_w - pad_w;
          int hend = hstart + kernel_h < in_h + pad_h ? hstart + kernel_h : in_h + pad_h;
          int wend = wstart + kernel_w < in_w + pad_w ? wstart + kernel_w : in_w + pad_w;
          int pool_size = (hend - hstart) * (wend - wstart);
          if (hstart < 0) hstart = 0;
          if (wstart < 0) wstart = 0;
          if (hend > in_h) hend = in_h;
          if (wend > in_w) wend = in_w;
          float max_val = -FLT_MAX, sum_val = 0.f;
          for (int ph = hstart; ph < hend; ++ph) {
            for (int pw = wstart; pw < wend; ++pw) {
              float value = in[ph * in_w + pw];
              max_val = std_max(max_val, value);
              sum_val += value;
            }
          }
          *out++ = (pool_type == 0) ? max_val : sum_val / pool_size;
        }
      }
    }
  }
}

/* ---- shadow/operators/kernels/pooling.cpp:44-86  Vision::Pooling3D ---- */
API void orc_pooling3d(const float* in, const int* in_shape, int pool_type, int kernel_d,
                       int kernel_h, int kernel_w, int stride_d, int stride_h, int stride_w,
                       int pad_d, int pad_h, int pad_w, const int* out_shape, float* out) {
  int batch = in_shape[0], channel = in_shape[1];
  int in_d = in_shape[2], in_h = in_shape[3], in_w = in_shape[4];
  int out_d = out_shape[2], out_h = out_shape[3], out_w = out_shape[4];
  for (int b = 0; b < batch; ++b) {
    for (int c = 0; c < channel; ++c, in += in_d * in_h * in_w) {
      for (int d = 0; d < out_d; ++d) {
        for (int h = 0; h < out_h; ++h) {
          for (int w = 0; w < out_w; ++w) {
            int dstart = d * stride_d - pad_d, hstart = h * stride_h - pad_h,
                wstart = w * stride_w - pad_w;
            int dend = dstart + kernel_d < in_d + pad_d ? dstart + kernel_d : in_d + pad_d;
            int hend = hstart + kernel_h < in_h + pad_h ? hstart + kernel_h : in_h + pad_h;
            int wend = wstart + kernel_w < in_w + pad_w ? wstart + kernel_w : in_w + pad_w;
            int pool_size = (dend - dstart) * (hend - hstart) * (wend - wstart);
            if (dstart < 0) dstart = 0;
            if (hstart < 0) hstart = 0;
            if (wstart < 0) wstart = 0;
            if (dend > in_d) dend = in_d;
            if (hend > in_h) hend = in_h;
            if (wend > in_w) wend = in_w;
            float max_val = -FLT_MAX, sum_val = 0.f;
            for (int pd = dstart; pd < dend; ++pd) {
              for (int ph = hstart; ph < hend; ++ph) {
                for (int pw = wstart; pw < wend; ++pw) {
                  float value = in[(pd * in_h + ph) * in_w + pw];
                  max_val = std_max(max_val, value);
                  sum_val += value;
                }
              }
            }
            *out++ = (pool_type == 0) ? max_val : sum_val / pool_size;
          }
        }
      }
    }
  }
}

/* ---- shadow/operators/pooling_op.cpp:7-17  pooling_out_size (fp32 arithmetic) ---- */
API int orc_pooling_out_size(int dim, int kernel_size, int stride, int pad, int full_pooling) {
  float t = (dim + 2.f * pad - kernel_size) / stride;
  return (int)((full_pooling ? ceilf(t) : floorf(t)) + 1);
}

/* ---- shadow/core/blas.cpp:238-247, 281-285  BlasSgemv, no-transpose plain-loop
 *      branch: y *= beta, then y[i] += (float) sum_fp64_j(alpha * A[i][j] * x[j])
 *      with the products formed in fp32.  Used here only as the row mean of the
 *      normalisation kernels (x = ones, beta = 0). ---- */
API void orc_sgemv_n(int M, int N, float alpha, const float* A, const float* x, float beta,
                     float* y) {
  for (int i = 0; i < M; ++i) y[i] *= beta;
  for (int i = 0; i < M; ++i) {
    double sum = 0;
    for (int j = 0; j < N; ++j) sum += alpha * A[i * N + j] * x[j];
    y[i] += (float)sum;
  }
}

/* ---- shadow/operators/kernels/group_norm.cpp:7-16  SubtractMeanAndSquare ---- */
API void orc_subtract_mean_and_square(const float* in, const float* mean, int count,
                                      int inner_num, float* out, float* square) {
  for (int i = 0; i < count; ++i) {
    float val = in[i] - mean[i / inner_num];
    out[i] = val;
    square[i] = val * val;
  }
}

/* ---- shadow/operators/kernels/group_norm.cpp:18-27  DivideVariance ---- */
API void orc_divide_variance(const float* in, const float* variance, int count, int inner_num,
                             float eps, float* out) {
  for (int i = 0; i < count; ++i) out[i] = in[i] / sqrtf(variance[i / inner_num] + eps);
}

/* ---- shadow/operators/kernels/group_norm.hpp:41-74 (GroupNorm, InstanceNorm) and
 *      layer_norm.hpp:22-57 (LayerNorm): the kernel classes' sequence of calls on
 *      x viewed as [outer_num][inner_num], without the trailing ScaleBias.
 *      mean / variance / temp are caller scratch of outer, outer, count floats,
 *      zero-filled like a fresh temp buffer. ---- */
API void orc_normalize_rows(const float* in, int outer_num, int inner_num, float eps, float* mean,
                            float* variance, float* temp, float* out) {
  int count = outer_num * inner_num;
  float* ones = (float*)malloc(sizeof(float) * (size_t)(inner_num > 0 ? inner_num : 1));
  orc_set(inner_num, 1, ones);
  orc_sgemv_n(outer_num, inner_num, 1.f / inner_num, in, ones, 0, mean);
  orc_subtract_mean_and_square(in, mean, count, inner_num, out, temp);
  orc_sgemv_n(outer_num, inner_num, 1.f / inner_num, temp, ones, 0, variance);
  orc_divide_variance(out, variance, count, inner_num, eps, out);
  free(ones);
}

/* ======================================================================
 * Data movers.
 * ====================================================================== */

/* ---- shadow/operators/kernels/concat.cpp:5-16  Vision::Concat (one input) ---- */
API void orc_concat(const float* in, int num_concats, int concat_size, int out_concat_axis,
                    int in_concat_axis, int offset_concat_axis, float* out) {
  for (int n = 0; n < num_concats; ++n)
    memcpy(out + (n * out_concat_axis + offset_concat_axis) * concat_size,
           in + n * in_concat_axis * concat_size, (size_t)in_concat_axis * concat_size * sizeof(float));
}

/* ---- shadow/operators/kernels/slice.cpp:5-16  Vision::Slice (one output) ---- */
API void orc_slice(const float* in, int num_slices, int slice_size, int in_slice_axis,
                   int out_slice_axis, int offset_slice_axis, float* out) {
  for (int n = 0; n < num_slices; ++n)
    memcpy(out + n * out_slice_axis * slice_size,
           in + (n * in_slice_axis + offset_slice_axis) * slice_size,
           (size_t)out_slice_axis * slice_size * sizeof(float));
}

/* ---- shadow/operators/kernels/stack.cpp:5-14  Vision::Stack (one input) ---- */
API void orc_stack(const float* in, int num_stacks, int stack_size, int out_stack_axis,
                   int offset_stack_axis, float* out) {
  for (int n = 0; n < num_stacks; ++n)
    memcpy(out + (n * out_stack_axis + offset_stack_axis) * stack_size, in + n * stack_size,
           (size_t)stack_size * sizeof(float));
}

/* ---- shadow/operators/kernels/gather.cpp:5-17  Vision::Gather ---- */
API void orc_gather(const float* in, const int* indexes, int num_indexes, int gather_dim,
                    int inner_num, int count, float* out) {
  int gather_num = num_indexes * inner_num;
  for (int i = 0; i < count; ++i) {
    int gather_index = indexes[(i / inner_num) % num_indexes];
    int in_index = (gather_index + i / gather_num * gather_dim) * inner_num + i % inner_num;
    out[i] = in[in_index];
  }
}

/* ---- shadow/operators/kernels/pad.cpp:5-32  Vision::Pad, after the Blas::Set fill of
 *      shadow/operators/kernels/pad.hpp:33-36; paddings = top, bottom, left, right,
 *      negative values crop ---- */
API void orc_pad(const float* in, const int* in_shape, const int* paddings, const int* out_shape,
                 float value, float* out) {
  int batch = in_shape[0], channel = in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  int out_h = out_shape[2], out_w = out_shape[3];
  orc_set(batch * channel * out_h * out_w, value, out);
  for (int b = 0; b < batch; ++b) {
    for (int c = 0; c < channel; ++c) {
      for (int h = 0; h < in_h; ++h) {
        if (h + paddings[0] < 0 || h >= in_h + paddings[1]) continue;
        int copy_w = in_w + (paddings[2] < 0 ? paddings[2] : 0) + (paddings[3] < 0 ? paddings[3] : 0);
        int in_offset = ((b * channel + c) * in_h + h) * in_w;
        int out_offset = ((b * channel + c) * out_h + h + paddings[0]) * out_w;
        if (paddings[2] < 0) in_offset -= paddings[2];
        else out_offset += paddings[2];
        memcpy(out + out_offset, in + in_offset, (size_t)copy_w * sizeof(float));
      }
    }
  }
}

/* ---- shadow/operators/kernels/permute.cpp:5-20  Vision::Permute with the step tables of
 *      shadow/operators/kernels/permute.hpp:33-43 ---- */
API void orc_permute(const float* in, int count, int num_axes, const int* order,
                     const int* old_steps, const int* new_steps, float* out) {
  for (int i = 0; i < count; ++i) {
    int old_idx = 0, idx = i;
    for (int j = 0; j < num_axes; ++j) {
      old_idx += (idx / new_steps[j]) * old_steps[order[j]];
      idx %= new_steps[j];
    }
    out[i] = in[old_idx];
  }
}

/* ---- shadow/operators/kernels/reorg.cpp:5-72  type 0 darknet, 1 natural ---- */
API int orc_reorg(const float* in, const int* in_shape, int type, int stride, float* out) {
  int batch = in_shape[0], in_c = in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  if (type == 0) {
    int out_c = in_c / (stride * stride);
    for (int b = 0; b < batch; ++b)
      for (int c = 0; c < in_c; ++c)
        for (int h = 0; h < in_h; ++h)
          for (int w = 0; w < in_w; ++w) {
            int c2 = c % out_c, offset = c / out_c;
            int h2 = h * stride + offset / stride, w2 = w * stride + offset % stride;
            int in_index = ((b * in_c + c) * in_h + h) * in_w + w;
            int out_index = ((b * out_c + c2) * in_h * stride + h2) * in_w * stride + w2;
            out[in_index] = in[out_index];
          }
  } else if (type == 1) {
    int out_c = in_c * stride * stride, out_h = in_h / stride, out_w = in_w / stride;
    for (int b = 0; b < batch; ++b)
      for (int c = 0; c < out_c; ++c)
        for (int h = 0; h < out_h; ++h)
          for (int w = 0; w < out_w; ++w) {
            int offset = c / stride, c2 = offset / stride;
            int h2 = h * stride + offset % stride, w2 = w * stride + c % stride;
            int in_index = ((b * in_c + c2) * in_h + h2) * in_w + w2;
            int out_index = ((b * out_c + c) * out_h + h) * out_w + w;
            out[out_index] = in[in_index];
          }
  } else {
    return -1;
  }
  return 0;
}

/* ---- shadow/operators/kernels/shuffle_channel.cpp:5-21 ---- */
API void orc_shuffle_channel(const float* in, int batch, int channel, int spatial_dim, int group,
                             float* out) {
  int num = channel * spatial_dim, group_column = channel / group;
  for (int b = 0; b < batch; ++b, in += num, out += num)
    for (int c = 0; c < channel; ++c) {
      int c_out = (c % group_column) * group + c / group_column;
      memcpy(out + c_out * spatial_dim, in + c * spatial_dim, (size_t)spatial_dim * sizeof(float));
    }
}

/* ---- shadow/operators/kernels/resize.cpp:5-27  ResizeNearest2D ---- */
API void orc_resize_nearest(const float* in, const int* in_shape, const int* out_shape, float* out) {
  int outer_num = in_shape[0] * in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  int out_h = out_shape[2], out_w = out_shape[3];
  float fh = (float)in_h / out_h, fw = (float)in_w / out_w;
  for (int n = 0; n < outer_num; ++n, in += in_h * in_w)
    for (int h = 0; h < out_h; ++h) {
      int src_h = (int)(h * fh);
      for (int w = 0; w < out_w; ++w) {
        int src_w = (int)(w * fw);
        *out++ = in[src_h * in_w + src_w];
      }
    }
}

/* ---- shadow/operators/kernels/resize.cpp:29-78  ResizeBilinear2D ---- */
API void orc_resize_bilinear(const float* in, const int* in_shape, int align_corners,
                             const int* out_shape, float* out) {
  int outer_num = in_shape[0] * in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  int out_h = out_shape[2], out_w = out_shape[3];
  float fh = align_corners ? (float)(in_h - 1) / (out_h - 1) : (float)in_h / out_h;
  float fw = align_corners ? (float)(in_w - 1) / (out_w - 1) : (float)in_w / out_w;
  for (int n = 0; n < outer_num; ++n, in += in_h * in_w) {
    for (int h = 0; h < out_h; ++h) {
      float src_h_f;
      if (align_corners) {
        src_h_f = h * fh;
      } else {
        src_h_f = (h + 0.5f) * fh - 0.5f;
        src_h_f = src_h_f < 0 ? 0 : src_h_f;
      }
      int src_h_l = (int)src_h_f, src_h_h = src_h_l + 1;
      if (src_h_l >= in_h - 1) src_h_h = src_h_l = in_h - 1;
      float sh = src_h_f - src_h_l;
      for (int w = 0; w < out_w; ++w) {
        float src_w_f;
        if (align_corners) {
          src_w_f = w * fw;
        } else {
          src_w_f = (w + 0.5f) * fw - 0.5f;
          src_w_f = src_w_f < 0 ? 0 : src_w_f;
        }
        int src_w_l = (int)src_w_f, src_w_h = src_w_l + 1;
        if (src_w_l >= in_w - 1) src_w_h = src_w_l = in_w - 1;
        float sw = src_w_f - src_w_l;
        int i0 = src_h_l * in_w + src_w_l, i1 = src_h_h * in_w + src_w_l;
        int i2 = src_h_l * in_w + src_w_h, i3 = src_h_h * in_w + src_w_h;
        *out++ = (1 - sh) * (1 - sw) * in[i0] + sh * (1 - sw) * in[i1] + (1 - sh) * sw * in[i2] +
                 sh * sw * in[i3];
      }
    }
  }
}

/* ---- shadow/operators/kernels/lrn.cpp:9-60  Vision::LRN across channels: per position
 *      a running fp32 sum of squares over the channels (add the entering one, then
 *      subtract the leaving one), scale = k + sum * (alpha / size), and a second pass
 *      out = in * powf(scale, -beta).  in_c >= (size - 1) / 2 is assumed, as by the
 *      reference (fewer channels make its third loop write in front of the buffer). ---- */
API void orc_lrn(const float* in, const int* in_shape, int size, float alpha, float beta, float k,
                 float* scale, float* out) {
  int batch = in_shape[0], in_c = in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  int step = in_h * in_w, count = batch * in_c * step;
  int pre_pad = (size - 1) / 2, post_pad = size - pre_pad - 1;
  float alpha_over_size = alpha / size;
  for (int b = 0; b < batch; ++b) {
    for (int h = 0; h < in_h; ++h) {
      for (int w = 0; w < in_w; ++w) {
        int offset = (b * in_c * in_h + h) * in_w + w, head = 0;
        const float* in_off = in + offset;
        float* scale_off = scale + offset;
        float accum_scale = 0.f;
        while (head < post_pad && head < in_c) {
          accum_scale += in_off[head * step] * in_off[head * step];
          head++;
        }
        while (head < in_c) {
          accum_scale += in_off[head * step] * in_off[head * step];
          if (head - size >= 0) accum_scale -= in_off[(head - size) * step] * in_off[(head - size) * step];
          scale_off[(head - post_pad) * step] = k + accum_scale * alpha_over_size;
          head++;
        }
        while (head < in_c + post_pad) {
          if (head - size >= 0) accum_scale -= in_off[(head - size) * step] * in_off[(head - size) * step];
          scale_off[(head - post_pad) * step] = k + accum_scale * alpha_over_size;
          head++;
        }
      }
    }
  }
  for (int i = 0; i < count; ++i) out[i] = in[i] * powf(scale[i], -beta);
}

/* ---- shadow/operators/kernels/grid_sample.cpp:9-100  Vision::GridSample ----
 * grid holds (x, y) in [-1, 1] per output position; (v + 1) / 2 * (extent - 1) is the
 * source coordinate.  mode 0: the nearest source cell (roundf, then the conversion to
 * int), mode 1: the four cells around the coordinate, weights in the reference's order
 * of operations.  padding_mode 0: outside the input reads as 0; 1: coordinates are
 * clamped to the border.
 * Where the reference leaves the value to the machine this follows what its x86-64
 * build does: a float that does not fit an int converts to INT_MIN.  A NaN coordinate
 * in mode 1 makes the reference index far outside its input; here it gives NaN. */
static int to_int_x86(float v) {
  return (v >= -2147483648.f && v < 2147483648.f) ? (int)v : (-2147483647 - 1);
}

API void orc_grid_sample(const float* in, const int* in_shape, const float* grid, int mode,
                         int padding_mode, const int* out_shape, float* out) {
  int batch = in_shape[0], channel = in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  int out_h = out_shape[2], out_w = out_shape[3];
  for (int b = 0; b < batch; ++b) {
    for (int c = 0; c < channel; ++c) {
      for (int h = 0; h < out_h; ++h) {
        for (int w = 0; w < out_w; ++w) {
          int grid_offset = ((b * out_h + h) * out_w + w) * 2;
          float x = grid[grid_offset], y = grid[grid_offset + 1];
          if (mode == 0) {
            int src_h = to_int_x86(roundf((y + 1) / 2.f * (in_h - 1)));
            int src_w = to_int_x86(roundf((x + 1) / 2.f * (in_w - 1)));
            if (padding_mode == 1) {
              src_h = src_h < 0 ? 0 : (src_h > in_h - 1 ? in_h - 1 : src_h);
              src_w = src_w < 0 ? 0 : (src_w > in_w - 1 ? in_w - 1 : src_w);
            } else if (src_h < 0 || src_w < 0 || src_h > in_h - 1 || src_w > in_w - 1) {
              *out++ = 0.f;
              continue;
            }
            *out++ = in[((b * channel + c) * in_h + src_h) * in_w + src_w];
            continue;
          }
          float src_h_f = (y + 1) / 2.f * (in_h - 1);
          float src_w_f = (x + 1) / 2.f * (in_w - 1);
          if (padding_mode == 1) {
            src_h_f = std_min(std_max(src_h_f, 0.f), in_h - 1.f);
            src_w_f = std_min(std_max(src_w_f, 0.f), in_w - 1.f);
          } else if (src_h_f < 0 || src_w_f < 0 || src_h_f > in_h - 1 || src_w_f > in_w - 1) {
            *out++ = 0.f;
            continue;
          }
          if (src_h_f != src_h_f || src_w_f != src_w_f) {
            *out++ = NAN;
            continue;
          }
          int src_h_0 = (int)floorf(src_h_f), src_h_1 = (int)ceilf(src_h_f);
          int src_w_0 = (int)floorf(src_w_f), src_w_1 = (int)ceilf(src_w_f);
          src_h_0 = src_h_0 < 0 ? 0 : src_h_0;
          src_h_1 = src_h_1 > in_h - 1 ? in_h - 1 : src_h_1;
          src_w_0 = src_w_0 < 0 ? 0 : src_w_0;
          src_w_1 = src_w_1 > in_w - 1 ? in_w - 1 : src_w_1;
          float sh = src_h_f - src_h_0, sw = src_w_f - src_w_0;
          int h_offset = (b * channel + c) * in_h;
          int i0 = (h_offset + src_h_0) * in_w + src_w_0, i1 = (h_offset + src_h_1) * in_w + src_w_0;
          int i2 = (h_offset + src_h_0) * in_w + src_w_1, i3 = (h_offset + src_h_1) * in_w + src_w_1;
          *out++ = (1 - sh) * (1 - sw) * in[i0] + sh * (1 - sw) * in[i1] + (1 - sh) * sw * in[i2] +
                   sh * sw * in[i3];
        }
      }
    }
  }
}
