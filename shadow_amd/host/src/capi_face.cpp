// C facade over the inner free-function layer, Blas::X<kGPU, float> and
// Vision::X<kGPU, float>, which the reference's kernels outside this path call
// directly (conv / connected epilogues, Eltwise, SSDNormalize).  Each function
// uploads host arrays into device buffers of the workspace's context, runs the
// call sequence exactly as the cited reference lines write it, and reads the
// result back.  Errors are reported like the rest of the facade (capi.cpp).
#include <cmath>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "shadow/blas.hpp"
#include "shadow/kernels/activate.hpp"
#include "shadow/kernels/scale.hpp"
#include "shadow/kernels/ssd_normalize.hpp"
#include "shadow/workspace.hpp"

using namespace Shadow;

extern "C" int shdw_host_set_error(const char* text);

namespace {

constexpr DeviceType G = DeviceType::kGPU;

template <typename F>
int guarded(F&& body) {
  try {
    body();
    return 0;
  } catch (const std::exception& e) {
    shdw_host_set_error(e.what());
    return -1;
  }
}

// A device buffer of `count` floats, optionally filled from the host.
class DeviceFloats {
 public:
  DeviceFloats(Context* ctx, size_t count, const float* host = nullptr) : ctx_(ctx), count_(count) {
    ptr_ = static_cast<float*>(ctx->allocator()->malloc((count ? count : 1) * sizeof(float), nullptr));
    if (host != nullptr && count > 0) ctx->allocator()->write(count * sizeof(float), host, ptr_);
  }
  ~DeviceFloats() {
    ctx_->synchronize();
    ctx_->allocator()->free(ptr_);
  }
  float* get() const { return ptr_; }
  void read(float* host) const {
    ctx_->allocator()->read(count_ * sizeof(float), ptr_, host);
    ctx_->synchronize();
  }

 private:
  Context* ctx_;
  size_t count_;
  float* ptr_ = nullptr;
};

typedef void (*Unary)(int, const float*, int, float*, int, Context*);
typedef void (*Binary)(int, const float*, int, const float*, int, float*, int, Context*);
typedef void (*Scalar)(int, const float*, int, float, float*, int, Context*);

struct Entry {
  const char* name;
  Unary unary;
  Binary binary;
  Scalar scalar;
};

#define SHDW_U(n) {#n, &Blas::n<G, float>, nullptr, nullptr}
#define SHDW_B(n) {#n, nullptr, &Blas::n<G, float>, &Blas::n<G, float>}
const Entry kTable[] = {SHDW_B(Add), SHDW_B(Sub), SHDW_B(Mul), SHDW_B(Div), SHDW_B(Pow), SHDW_B(Max), SHDW_B(Min),
                        SHDW_U(Abs), SHDW_U(Square), SHDW_U(Sqrt), SHDW_U(Log), SHDW_U(Exp), SHDW_U(Sin),
                        SHDW_U(Cos), SHDW_U(Tan), SHDW_U(Asin), SHDW_U(Acos), SHDW_U(Atan), SHDW_U(Floor),
                        SHDW_U(Ceil), SHDW_U(Neg), SHDW_U(Reciprocal)};
#undef SHDW_U
#undef SHDW_B

}  // namespace

extern "C" {

// One Blas::<name><kGPU, float> call with element offsets, the way the reference
// passes them (e.g. Blas::Mul(num, in_data, offset, alpha, out_data, offset, ctx),
// shadow/operators/kernels/ssd_normalize.hpp:55-56).
//   a      : a_count floats, uploaded whole; the call reads a + offa.  nullptr makes
//            the y buffer the first operand as well (in place when offa == offy)
//   b      : nullptr selects the scalar form of a binary function (with alpha)
//   y_io   : y_count floats, uploaded first (so that untouched cells can be told
//            apart) and read back whole; the call writes y + offy
// name: Add Sub Mul Div Pow Max Min (tensor or scalar form), the 15 unary names,
// Set (alpha), Sscal (alpha, in place on y), Scopy, Saxpy (alpha), Sasum (the host
// result goes to y_io[0], the device buffer is not touched).
int shdw_host_face_blas(void* ws, const char* name, int n, const float* a, int a_count, int offa,
                        const float* b, int b_count, int offb, float alpha, float* y_io, int y_count,
                        int offy) {
  return guarded([&] {
    Context* ctx = static_cast<Workspace*>(ws)->Ctx().get();
    CHECK_NOTNULL(ctx);
    const std::string fn(name ? name : "");
    DeviceFloats da(ctx, a_count, a), db(ctx, b_count, b), dy(ctx, y_count, y_io);
    bool done = false;
    const float* first = a != nullptr ? da.get() : dy.get();
    for (const Entry& e : kTable) {
      if (fn != e.name) continue;
      if (e.unary != nullptr) e.unary(n, first, offa, dy.get(), offy, ctx);
      else if (b != nullptr) e.binary(n, first, offa, db.get(), offb, dy.get(), offy, ctx);
      else e.scalar(n, first, offa, alpha, dy.get(), offy, ctx);
      done = true;
    }
    if (fn == "Set") {
      Blas::Set<G, float>(n, alpha, dy.get(), offy, ctx);
    } else if (fn == "Sscal") {
      Blas::BlasSscal<G, float>(n, alpha, dy.get(), offy, ctx);
    } else if (fn == "Scopy") {
      Blas::BlasScopy<G, float>(n, da.get(), offa, dy.get(), offy, ctx);
    } else if (fn == "Saxpy") {
      Blas::BlasSaxpy<G, float>(n, alpha, da.get(), offa, dy.get(), offy, ctx);
    } else if (fn == "Sasum") {
      float sum = 0;
      Blas::BlasSasum<G, float>(n, da.get(), offa, &sum, ctx);
      y_io[0] = sum;
      return;
    } else {
      CHECK(done) << "unknown Blas function " << fn;
    }
    dy.read(y_io);
  });
}

// The convolution epilogue, shadow/operators/kernels/conv.hpp:122-131:
//   Vision::Bias(out, count, bias, num_output, out_spatial_dim, out)   in place
//   Vision::Activate(out, out, count, 1, 0)                            in place
// activate_type other than 1 skips the second call, as the reference does.
int shdw_host_face_conv_epilogue(void* ws, float* out_io, int count, const float* bias, int num_output,
                                 int out_spatial_dim, int bias_term, int activate_type) {
  return guarded([&] {
    Context* ctx = static_cast<Workspace*>(ws)->Ctx().get();
    DeviceFloats dout(ctx, count, out_io), dbias(ctx, num_output, bias);
    float* out_data = dout.get();
    if (bias_term) {
      Vision::Bias<G, float>(out_data, count, dbias.get(), num_output, out_spatial_dim, out_data, ctx);
    }
    if (activate_type == 1) {
      Vision::Activate<G, float>(out_data, out_data, count, activate_type, 0, ctx);
    }
    dout.read(out_io);
  });
}

// Eltwise SUM as the reference's kernel class writes it, shadow/operators/kernels/
// eltwise.hpp:37-44: Blas::Set(count, 0, out) and one Blas::BlasSaxpy per input.
int shdw_host_face_eltwise_sum(void* ws, int k, const float* const* inputs, const float* coeff, int count,
                               float* out) {
  return guarded([&] {
    Context* ctx = static_cast<Workspace*>(ws)->Ctx().get();
    std::vector<std::unique_ptr<DeviceFloats>> in;
    for (int n = 0; n < k; ++n) in.emplace_back(new DeviceFloats(ctx, count, inputs[n]));
    DeviceFloats dout(ctx, count);
    float* out_data = dout.get();
    Blas::Set<G, float>(count, 0, out_data, 0, ctx);
    for (int n = 0; n < k; ++n) {
      Blas::BlasSaxpy<G, float>(count, coeff[n], in[n]->get(), 0, out_data, 0, ctx);
    }
    dout.read(out);
  });
}

// SSDNormalizeKernelDefault<kGPU>::Run as written in shadow/operators/kernels/
// ssd_normalize.hpp:47-75: Square, then per item BlasSasum (a host value) and the
// scalar Mul with offsets, or the per-position kernel; then BlasSscal with the
// shared scale read back to the host, or Vision::Scale per channel.
int shdw_host_face_ssd_normalize(void* ws, const float* in, int batch, int channel, int spatial_dim,
                                 int across_spatial, int channel_shared, float eps, const float* scale,
                                 float* out) {
  return guarded([&] {
    Context* ctx = static_cast<Workspace*>(ws)->Ctx().get();
    const int num = channel * spatial_dim, count = batch * num;
    DeviceFloats din(ctx, count, in), dout(ctx, count);
    const float* in_data = din.get();
    float* out_data = dout.get();

    Blas::Square<G, float>(count, in_data, 0, out_data, 0, ctx);

    if (across_spatial) {
      for (int b = 0; b < batch; ++b) {
        int offset = b * num;
        float sum = 0;
        Blas::BlasSasum<G, float>(num, out_data, offset, &sum, ctx);
        Blas::Mul<G, float>(num, in_data, offset, 1.f / std::sqrt(sum + eps), out_data, offset, ctx);
      }
    } else {
      // the reference's per-position kernel with its [batch, spatial_dim] scratch blob;
      // here the same device call without a scale
      Vision::SSDNormalize<G, float>(in_data, batch, channel, spatial_dim, false, eps, nullptr, false,
                                     nullptr, out_data, ctx);
    }

    if (scale != nullptr) {
      if (channel_shared) {
        Blas::BlasSscal<G, float>(count, scale[0], out_data, 0, ctx);
      } else {
        DeviceFloats dscale(ctx, channel, scale);
        Vision::Scale<G, float>(out_data, count, dscale.get(), channel, spatial_dim, out_data, ctx);
        dout.read(out);  // before dscale goes away
        return;
      }
    }
    dout.read(out);
  });
}

}  // extern "C"
