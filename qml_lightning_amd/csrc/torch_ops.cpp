// libqmll_torch.so: the reference's TorchScript operator libraries, over the C ABI of libqmll.
//
// The reference registers its operators from C++ with TORCH_LIBRARY
// (qml_lightning/cuda/torchscript/FCHL19.cpp:318-333, SORF.cpp:138-150), which is what lets a
// saved model run wherever libtorch runs, Python or not.  This file does the same for the
// HIP kernels: every operator below takes and returns tensors, validates them, allocates the
// outputs, and forwards device pointers and the current HIP stream to include/qmll.h.  The
// autograd formulas are those of the reference's Function classes (FCHL19.cpp:241-316,
// SORF.cpp:74-136); the additional fused operators (element sort, typed projection, fused
// SORF / RFF energy) return d(energy)/d(input) from their forward kernel and only scale it
// in backward.
//
// Host code only: no kernels here.  Loaded with torch.ops.load_library (Python) or as a
// shared library by a C++ host; it pulls in libqmll.so from its own directory.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/autograd.h>
#include <torch/library.h>

#include <functional>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/qmll.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::Function;
using torch::autograd::variable_list;

void* stream() { return (void*)c10::hip::getCurrentHIPStream().stream(); }

void check(int rc, const char* who) {
    if (rc != QMLL_OK) {
        const char* msg = qmll_last_error();
        TORCH_CHECK(false, (msg && msg[0]) ? std::string(msg) : std::string(who) + " failed");
    }
}

// same fault, same exception as the reference's TORCH_CHECK (fchl_cuda.cpp:30-34)
void need_cuda(const Tensor& t, const char* name) { TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor"); }

Tensor f32(const Tensor& t) { return t.scalar_type() == at::kFloat ? t.contiguous() : t.to(at::kFloat).contiguous(); }
Tensor i32(const Tensor& t) { return t.scalar_type() == at::kInt ? t.contiguous() : t.to(at::kInt).contiguous(); }

const float* fp(const Tensor& t) { return t.defined() && t.numel() ? t.data_ptr<float>() : nullptr; }
const int* ip(const Tensor& t) { return t.defined() && t.numel() ? t.data_ptr<int>() : nullptr; }

float scalar(const Tensor& t) { return t.item<float>(); }

// Model constants that a kernel wants in a prepared form (fp32 operands split into fp16 parts): prepared
// once per tensor and kept until the tensor dies, is written to in place or changes its storage.
struct Prepared {
    c10::weak_intrusive_ptr<c10::TensorImpl> owner;
    int64_t version;
    const void* data;
    Tensor buffer;
};
std::mutex prepared_mutex;
std::map<std::pair<const c10::TensorImpl*, int>, Prepared> prepared;

int64_t version_of(const Tensor& t) { return t.is_inference() ? -1 : (int64_t)t._version(); }

Tensor prepared_form(const Tensor& t, int kind, const std::function<Tensor(const Tensor&)>& make) {
    std::lock_guard<std::mutex> lock(prepared_mutex);
    const auto key = std::make_pair((const c10::TensorImpl*)t.unsafeGetTensorImpl(), kind);
    auto it = prepared.find(key);
    if (it != prepared.end()) {
        auto alive = it->second.owner.lock();
        if (alive && alive.get() == t.unsafeGetTensorImpl() && it->second.version == version_of(t) &&
            it->second.data == t.const_data_ptr())
            return it->second.buffer;
        prepared.erase(it);
    }
    if (prepared.size() >= 64) {      // forget tensors that are gone
        for (auto e = prepared.begin(); e != prepared.end();) e = e->second.owner.expired() ? prepared.erase(e) : std::next(e);
    }
    Tensor buffer = make(t);
    prepared.emplace(key, Prepared{c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr()), version_of(t),
                                   t.const_data_ptr(), buffer});
    return buffer;
}

// alpha as the kernels contract with it (fp32): a model stores it in fp64 (qml_lightning/models/kernel.py:226-234),
// and the conversion, a launch per call otherwise, is kept per tensor version like the other prepared constants
Tensor alpha32(const Tensor& alpha) {
    if (alpha.scalar_type() == at::kFloat) return alpha.contiguous();
    return prepared_form(alpha, 3, [](const Tensor& a) { return a.to(at::kFloat).contiguous(); });
}

// ---- FCHL19 -----------------------------------------------------------------------------
struct FchlInputs {
    Tensor X, types, cell, inv_cell, atomIDs, molIDs, natoms, Rs2, Rs3;
    qmll_fchl_params prm;
    int A, B, n, R;
};

Tensor element_types(const Tensor& X, const Tensor& Z, const Tensor& natoms, const Tensor& species) {
    need_cuda(X, "coordinates");
    need_cuda(Z, "charges");
    need_cuda(species, "species");
    Tensor Zb = f32(Z.dim() == 1 ? Z.unsqueeze(0) : Z);
    Tensor nat = i32(natoms), sp = f32(species);
    const int B = (int)Zb.size(0), n = (int)Zb.size(1);
    Tensor out = at::empty({B, n}, Zb.options().dtype(at::kInt));
    check(qmll_element_types(fp(Zb), ip(nat), fp(sp), B, n, (int)sp.size(0), out.data_ptr<int>(), stream()),
          "qmll_element_types");
    return out;
}

FchlInputs prepare(const Tensor& X, const Tensor& Z, const Tensor& species, const Tensor& atomIDs, const Tensor& molIDs,
                   const Tensor& atom_counts, const Tensor& cell, const Tensor& inv_cell, const Tensor& Rs2,
                   const Tensor& Rs3, const Tensor& eta2, const Tensor& eta3, const Tensor& two_body_decay,
                   const Tensor& three_body_weight, const Tensor& three_body_decay, const Tensor& rcut,
                   bool with_types = true) {
    need_cuda(X, "coordinates");   // torchscript/FCHL19.cpp:251-258
    need_cuda(Z, "charges");
    need_cuda(species, "species");
    need_cuda(atomIDs, "atomIDs");
    need_cuda(molIDs, "molIDs");
    need_cuda(atom_counts, "atom_counts");
    need_cuda(cell, "cell");
    need_cuda(inv_cell, "inv_cell");
    FchlInputs in;
    in.X = f32(X.dim() == 2 ? X.unsqueeze(0) : X);   // fchl_cuda.cpp:72-76
    in.natoms = i32(atom_counts);
    if (with_types) in.types = element_types(in.X, Z, in.natoms, species);
    if (cell.numel() > 0) {   // an empty [0,3,3] tensor means no periodic images
        in.cell = f32(cell);
        in.inv_cell = f32(inv_cell);
    }
    in.atomIDs = i32(atomIDs);
    in.molIDs = i32(molIDs);
    in.Rs2 = f32(Rs2);
    in.Rs3 = f32(Rs3);
    in.prm.nspecies = (int)species.size(0);
    in.prm.nRs2 = (int)in.Rs2.size(0);
    in.prm.nRs3 = (int)in.Rs3.size(0);
    in.prm.eta2 = scalar(eta2);
    in.prm.eta3 = scalar(eta3);
    in.prm.two_body_decay = scalar(two_body_decay);
    in.prm.three_body_weight = scalar(three_body_weight);
    in.prm.three_body_decay = scalar(three_body_decay);
    in.prm.rcut = scalar(rcut);
    in.A = (int)in.atomIDs.size(0);
    in.B = (int)in.X.size(0);
    in.n = (int)in.X.size(1);
    in.R = in.prm.nspecies * in.prm.nRs2 + in.prm.nspecies * (in.prm.nspecies + 1) * in.prm.nRs3;
    return in;
}

#define FCHL_TENSORS                                                                                             \
    const Tensor &X, const Tensor &Z, const Tensor &species, const Tensor &atomIDs, const Tensor &molIDs,        \
        const Tensor &atom_counts, const Tensor &cell, const Tensor &inv_cell, const Tensor &Rs2,                \
        const Tensor &Rs3, const Tensor &eta2, const Tensor &eta3, const Tensor &two_body_decay,                 \
        const Tensor &three_body_weight, const Tensor &three_body_decay, const Tensor &rcut
#define FCHL_PASS                                                                                                \
    X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3, two_body_decay,           \
        three_body_weight, three_body_decay, rcut
#define FCHL_ABI_T(in, types)                                                                                \
    fp(in.X), types, fp(in.cell), fp(in.inv_cell), ip(in.atomIDs), ip(in.molIDs), ip(in.natoms), nullptr,       \
        nullptr, 0, in.A, in.B, in.n, fp(in.Rs2), fp(in.Rs3), &in.prm
#define FCHL_ABI(in) FCHL_ABI_T(in, ip(in.types))

Tensor fchl_forwards_impl(FCHL_TENSORS) {
    FchlInputs in = prepare(FCHL_PASS);
    Tensor rep = at::zeros({in.B, in.n, in.R}, in.X.options());   // padded slots stay zero (fchl_cuda.cpp:83)
    check(qmll_fchl19_forward(FCHL_ABI(in), rep.data_ptr<float>(), stream()), "qmll_fchl19_forward");
    return rep;
}

Tensor fchl_backwards(const Tensor& grad, FCHL_TENSORS) {
    FchlInputs in = prepare(FCHL_PASS);
    Tensor g = f32(grad).reshape({in.B, in.n, in.R});
    Tensor gX = at::zeros({in.B, in.n, 3}, in.X.options());
    check(qmll_fchl19_vjp(FCHL_ABI(in), fp(g), gX.data_ptr<float>(), stream()), "qmll_fchl19_vjp");
    return gX.reshape(X.sizes());
}

std::vector<Tensor> get_fchl_and_derivative(FCHL_TENSORS, bool gradients) {
    FchlInputs in = prepare(FCHL_PASS);
    Tensor rep = at::zeros({in.B, in.n, in.R}, in.X.options());
    if (!gradients) {
        check(qmll_fchl19_forward(FCHL_ABI(in), rep.data_ptr<float>(), stream()), "qmll_fchl19_forward");
        return {rep};
    }
    Tensor jac = at::zeros({in.B, in.n, in.n, 3, in.R}, in.X.options());   // fchl_cuda.cpp:186-187
    check(qmll_fchl19_jacobian(FCHL_ABI(in), rep.data_ptr<float>(), jac.data_ptr<float>(), stream()),
          "qmll_fchl19_jacobian");
    return {rep, jac};
}

// autograd on X only (torchscript/FCHL19.cpp:241-316)
struct FchlFn : public Function<FchlFn> {
    static Tensor forward(AutogradContext* ctx, FCHL_TENSORS) {
        ctx->save_for_backward({FCHL_PASS});
        return fchl_forwards_impl(FCHL_PASS);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const variable_list s = ctx->get_saved_variables();
        variable_list out(16);
        if (grads[0].defined())
            out[0] = fchl_backwards(grads[0].contiguous(), s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], s[9],
                                    s[10], s[11], s[12], s[13], s[14], s[15]);
        return out;
    }
};

Tensor fchl_forwards(FCHL_TENSORS) { return FchlFn::apply(FCHL_PASS); }

Tensor get_num_neighbours(const Tensor& X, const Tensor& natoms, const Tensor& rcut, const Tensor& cell,
                          const Tensor& inv_cell) {
    need_cuda(X, "coordinates");
    Tensor Xb = f32(X.dim() == 2 ? X.unsqueeze(0) : X), nat = i32(natoms), c, ic;
    if (cell.numel() > 0) {
        c = f32(cell);
        ic = f32(inv_cell);
    }
    const int B = (int)Xb.size(0), n = (int)Xb.size(1);
    Tensor out = at::empty({B, n}, Xb.options().dtype(at::kInt));
    check(qmll_num_neighbours(fp(Xb), ip(nat), fp(c), fp(ic), B, n, scalar(rcut), out.data_ptr<int>(), stream()),
          "qmll_num_neighbours");
    return out;
}

Tensor get_neighbour_list(const Tensor& X, const Tensor& natoms, const Tensor& max_neighbours, const Tensor& rcut,
                          const Tensor& cell, const Tensor& inv_cell) {
    need_cuda(X, "coordinates");
    Tensor Xb = f32(X.dim() == 2 ? X.unsqueeze(0) : X), nat = i32(natoms), c, ic;
    if (cell.numel() > 0) {
        c = f32(cell);
        ic = f32(inv_cell);
    }
    const int B = (int)Xb.size(0), n = (int)Xb.size(1), nn = max_neighbours.item<int>();
    Tensor out = at::empty({B, n, nn}, Xb.options().dtype(at::kInt));
    check(qmll_neighbour_list(fp(Xb), ip(nat), fp(c), fp(ic), B, n, nn, scalar(rcut),
                              nn > 0 ? out.data_ptr<int>() : nullptr, stream()),
          "qmll_neighbour_list");
    return out;
}

// ---- SORF coefficients and cos features (the reference's two operators) --------------------
Tensor sorf_coefficients_impl(const Tensor& u, const Tensor& D, const Tensor& cn, const Tensor& nt) {
    need_cuda(u, "input");
    need_cuda(D, "dmatrix");
    Tensor uu = f32(u), DD = f32(D);
    const int A = (int)uu.size(0), d = (int)uu.size(1), S = (int)DD.size(1), T = nt.item<int>();   // SORF.cpp:85
    TORCH_CHECK(T <= DD.size(0), "ntransforms (", T, ") exceeds the ", DD.size(0), " diagonals given");
    TORCH_CHECK(uu.dim() == 2 && DD.dim() == 3 && DD.size(2) == d, "get_SORF_coefficients: input is [", uu.sizes(),
                "], diagonals are [", DD.sizes(), "]: the last dimensions must agree");
    Tensor out = at::empty({A, S, d}, uu.options());
    check(qmll_sorf_forward(fp(uu), fp(DD), A, d, S, T, scalar(cn), A ? out.data_ptr<float>() : nullptr, stream()),
          "qmll_sorf_forward");
    return out;
}

Tensor sorf_coefficients_backward(const Tensor& grad, const Tensor& D, const Tensor& cn, const Tensor& nt) {
    need_cuda(grad, "input");
    need_cuda(D, "dmatrix");
    Tensor g = f32(grad), DD = f32(D);
    const int A = (int)g.size(0), S = (int)g.size(1), d = (int)g.size(2), T = nt.item<int>();       // SORF.cpp:99
    TORCH_CHECK(T <= DD.size(0), "ntransforms (", T, ") exceeds the ", DD.size(0), " diagonals given");
    TORCH_CHECK(DD.dim() == 3 && DD.size(1) == S && DD.size(2) == d, "get_SORF_coefficients_backward: gradient is [",
                g.sizes(), "], diagonals are [", DD.sizes(), "]");
    Tensor out = at::empty({A, d}, g.options());
    check(qmll_sorf_adjoint(fp(g), fp(DD), A, d, S, T, scalar(cn), A ? out.data_ptr<float>() : nullptr, stream()),
          "qmll_sorf_adjoint");
    return out;
}

struct SorfFn : public Function<SorfFn> {
    static Tensor forward(AutogradContext* ctx, const Tensor& u, const Tensor& D, const Tensor& cn, const Tensor& nt) {
        ctx->save_for_backward({D, cn, nt});
        return sorf_coefficients_impl(u, D, cn, nt);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const variable_list s = ctx->get_saved_variables();
        variable_list out(4);
        if (grads[0].defined()) out[0] = sorf_coefficients_backward(grads[0].contiguous(), s[0], s[1], s[2]);
        return out;
    }
};

Tensor get_SORF_coefficients(const Tensor& u, const Tensor& D, const Tensor& cn, const Tensor& nt) {
    return SorfFn::apply(u, D, cn, nt);
}

Tensor cos_features_impl(const Tensor& coeffs, const Tensor& b, const Tensor& nmol_t, const Tensor& batch_indexes) {
    need_cuda(coeffs, "coeffs");
    need_cuda(b, "b");
    need_cuda(batch_indexes, "batch_indexes");
    Tensor c = f32(coeffs), bb = f32(b), idx = i32(batch_indexes);
    const int A = (int)c.size(0), F = (int)c.size(1), nmol = nmol_t.item<int>();                     // SORF.cpp:118
    TORCH_CHECK(bb.numel() == F && idx.numel() == A, "get_cos_features: coefficients are [", c.sizes(), "], bias has ",
                bb.numel(), " entries, batch_indexes ", idx.numel());
    Tensor out = at::zeros({nmol, F}, c.options());
    if (A == 0) return out;
    // segment table of the (ascending) molecule index, validated on the device
    Tensor seg = at::zeros({nmol + 2}, c.options().dtype(at::kInt));
    check(qmll_segment_offsets(ip(idx), A, nmol, seg.data_ptr<int>(), stream()), "qmll_segment_offsets");
    check(qmll_cos_features_f32(fp(c), fp(bb), ip(idx), ip(seg), A, F, nmol, out.data_ptr<float>(), stream()),
          "qmll_cos_features_f32");
    return out;
}

Tensor cos_features_backward(const Tensor& grad, const Tensor& coeffs, const Tensor& b, const Tensor& nmol_t,
                             const Tensor& batch_indexes) {
    Tensor g = f32(grad), c = f32(coeffs), bb = f32(b), idx = i32(batch_indexes);
    const int A = (int)c.size(0), F = (int)c.size(1), nmol = (int)g.size(0);
    (void)nmol_t;
    TORCH_CHECK(bb.numel() == F && idx.numel() == A && g.dim() == 2 && g.size(1) == F,
                "get_cos_features_backward: coefficients are [", c.sizes(), "], gradient [", g.sizes(), "], bias has ",
                bb.numel(), " entries, batch_indexes ", idx.numel());
    Tensor out = at::empty({A, F}, c.options());
    if (A == 0) return out;
    check(qmll_cos_features_backward(fp(g), fp(c), fp(bb), ip(idx), A, F, nmol, out.data_ptr<float>(), stream()),
          "qmll_cos_features_backward");
    return out;
}

struct CosFn : public Function<CosFn> {
    static Tensor forward(AutogradContext* ctx, const Tensor& coeffs, const Tensor& b, const Tensor& nmol,
                          const Tensor& batch_indexes) {
        ctx->save_for_backward({coeffs, b, nmol, batch_indexes});
        return cos_features_impl(coeffs, b, nmol, batch_indexes);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const variable_list s = ctx->get_saved_variables();
        variable_list out(4);
        if (grads[0].defined()) out[0] = cos_features_backward(grads[0].contiguous(), s[0], s[1], s[2], s[3]);
        return out;
    }
};

Tensor get_cos_features(const Tensor& coeffs, const Tensor& b, const Tensor& nmol, const Tensor& batch_indexes) {
    return CosFn::apply(coeffs, b, nmol, batch_indexes);
}

// ---- fused predict operators (not part of the reference's operator set) -------------------
// Each returns (energies, d energy / d input rows); backward scales the stored gradient rows
// by the incoming energy gradients.
Tensor empty_like_none(const Tensor& like) { return at::empty({0}, like.options()); }

std::tuple<Tensor, Tensor> sorf_energy_impl(const Tensor& sub, const Tensor& D, const Tensor& bias, const Tensor& alpha,
                                            const Tensor& cn, const Tensor& nt) {
    Tensor x = f32(sub), DD = f32(D), bb = f32(bias), al = alpha32(alpha);
    need_cuda(x, "sub");
    const int A = (int)x.size(0), d = (int)x.size(1), S = (int)DD.size(1), T = nt.item<int>();
    TORCH_CHECK(DD.dim() == 3 && DD.size(2) == d && T <= DD.size(0) && bb.numel() == (int64_t)S * d &&
                    al.numel() == (int64_t)S * d,
                "sorf_energy: x [", x.sizes(), "], diagonals [", DD.sizes(), "], bias ", bb.numel(), " and alpha ",
                al.numel(), " entries do not fit together");
    Tensor e = at::empty({A}, x.options()), gx = at::empty({A, d}, x.options());
    check(qmll_sorf_energy_fused(fp(x), fp(DD), fp(bb), fp(al), nullptr, A, d, S, T, scalar(cn),
                                 A ? e.data_ptr<float>() : nullptr, A ? gx.data_ptr<float>() : nullptr, stream()),
          "qmll_sorf_energy_fused");
    return {e, gx};
}

struct SorfEnergyFn : public Function<SorfEnergyFn> {
    static variable_list forward(AutogradContext* ctx, const Tensor& sub, const Tensor& D, const Tensor& bias,
                                 const Tensor& alpha, const Tensor& cn, const Tensor& nt) {
        auto r = sorf_energy_impl(sub, D, bias, alpha, cn, nt);
        ctx->save_for_backward({std::get<1>(r)});
        ctx->mark_non_differentiable({std::get<1>(r)});
        ctx->set_materialize_grads(false);
        return {std::get<0>(r), std::get<1>(r)};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        variable_list out(6);
        if (grads[0].defined()) out[0] = ctx->get_saved_variables()[0] * grads[0].unsqueeze(1);
        return out;
    }
};

std::tuple<Tensor, Tensor> sorf_energy(const Tensor& sub, const Tensor& D, const Tensor& bias, const Tensor& alpha,
                                       const Tensor& cn, const Tensor& nt) {
    auto r = SorfEnergyFn::apply(sub, D, bias, alpha, cn, nt);
    return {r[0], r[1]};
}

std::tuple<Tensor, Tensor> sorf_energy_typed_impl(const Tensor& x_all, const Tensor& types, const Tensor& atom_slots,
                                                  const Tensor& Dmat, const Tensor& bias, const Tensor& alpha,
                                                  const Tensor& cn, const Tensor& nt, bool with_grad) {
    Tensor x = f32(x_all), DD = f32(Dmat), bb = f32(bias), al = alpha32(alpha);
    need_cuda(x, "x_all");
    Tensor ty = i32(types).reshape({-1}), sl = i32(atom_slots);
    const int ne = (int)DD.size(0), Tn = (int)DD.size(1), S = (int)DD.size(2), d = (int)DD.size(3);
    const int N = (int)x.size(0), T = nt.item<int>();
    TORCH_CHECK(x.size(1) == (int64_t)ne * d && ty.size(0) == N, "sorf_energy_typed: x_all is [", x.size(0), ", ",
                x.size(1), "], expected [", ty.size(0), ", ", ne * d, "]");
    TORCH_CHECK(T == Tn, "sorf_energy_typed: ", Tn, " diagonals stored per stack, ", T, " transforms asked for");
    TORCH_CHECK(bb.dim() == 2 && bb.size(0) == ne && bb.size(1) == (int64_t)S * d && al.numel() == (int64_t)S * d,
                "sorf_energy_typed: bias [", bb.sizes(), "] / alpha with ", al.numel(), " entries do not fit ", ne,
                " elements and ", S * d, " features");
    Tensor e = at::zeros({N}, x.options());
    Tensor gx = with_grad ? at::zeros({N, (int64_t)ne * d}, x.options()) : empty_like_none(x);
    check(qmll_sorf_energy_typed(fp(x), ip(ty), ip(sl), fp(DD), fp(bb), fp(al), (int)sl.size(0), N, ne, d, S, T,
                                 scalar(cn), N ? e.data_ptr<float>() : nullptr,
                                 with_grad && N ? gx.data_ptr<float>() : nullptr, stream()),
          "qmll_sorf_energy_typed");
    return {e, gx};
}

struct SorfEnergyTypedFn : public Function<SorfEnergyTypedFn> {
    static variable_list forward(AutogradContext* ctx, const Tensor& x_all, const Tensor& types, const Tensor& atom_slots,
                                 const Tensor& Dmat, const Tensor& bias, const Tensor& alpha, const Tensor& cn,
                                 const Tensor& nt, bool with_grad) {
        auto r = sorf_energy_typed_impl(x_all, types, atom_slots, Dmat, bias, alpha, cn, nt, with_grad);
        ctx->save_for_backward({std::get<1>(r)});
        ctx->mark_non_differentiable({std::get<1>(r)});
        ctx->set_materialize_grads(false);
        return {std::get<0>(r), std::get<1>(r)};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        variable_list out(9);
        if (!grads[0].defined()) return out;
        const Tensor gx = ctx->get_saved_variables()[0];
        TORCH_CHECK(gx.numel() != 0, "sorf_energy_typed was called with with_grad=False but a gradient is requested");
        out[0] = gx * grads[0].unsqueeze(1);
        return out;
    }
};

std::tuple<Tensor, Tensor> sorf_energy_typed(const Tensor& x_all, const Tensor& types, const Tensor& atom_slots,
                                             const Tensor& Dmat, const Tensor& bias, const Tensor& alpha,
                                             const Tensor& cn, const Tensor& nt, bool with_grad) {
    auto r = SorfEnergyTypedFn::apply(x_all, types, atom_slots, Dmat, bias, alpha, cn, nt, with_grad);
    return {r[0], r[1]};
}

std::tuple<Tensor, Tensor> sort_by_type(const Tensor& types, const Tensor& slots, int64_t ne) {
    need_cuda(types, "types");
    Tensor ty = i32(types).reshape({-1}), sl = i32(slots).reshape({-1});
    const int A = (int)sl.size(0);
    Tensor sorted = at::empty({A}, ty.options()), offsets = at::empty({ne + 1}, ty.options());
    const size_t nbytes = qmll_sort_by_type_workspace(A, (int)ne);
    Tensor work = at::empty({(int64_t)std::max<size_t>(nbytes / 4, 1)}, ty.options());
    check(qmll_sort_by_type(ip(ty), ip(sl), A, (int)ne, work.data_ptr<int>(), nbytes,
                            A ? sorted.data_ptr<int>() : nullptr, offsets.data_ptr<int>(), stream()),
          "qmll_sort_by_type");
    return {sorted, offsets};
}

// sort_by_type of the listed atoms of a padded batch (slot = molIDs * n + atomIDs), one launch for small batches
std::tuple<Tensor, Tensor> sort_atoms_by_type(const Tensor& types, const Tensor& atomIDs, const Tensor& molIDs, int64_t n,
                                              int64_t ne) {
    need_cuda(types, "types");
    Tensor ty = i32(types).reshape({-1}), ai = i32(atomIDs).reshape({-1}), mi = i32(molIDs).reshape({-1});
    const int A = (int)ai.size(0);
    TORCH_CHECK(mi.size(0) == A, "sort_atoms_by_type: ", A, " atom indices, ", mi.size(0), " molecule indices");
    Tensor sorted = at::empty({A}, ty.options()), offsets = at::empty({ne + 1}, ty.options());
    const size_t nbytes = qmll_sort_atoms_workspace(A, (int)ne);
    Tensor work = nbytes ? at::empty({(int64_t)(nbytes / 4)}, ty.options()) : Tensor();
    check(qmll_sort_atoms_by_type(ip(ty), ip(ai), ip(mi), (int)n, A, (int)ne, nbytes ? work.data_ptr<int>() : nullptr, nbytes,
                                  A ? sorted.data_ptr<int>() : nullptr, offsets.data_ptr<int>(), stream()),
          "qmll_sort_atoms_by_type");
    return {sorted, offsets};
}

// the reductors prepared for the fp16 matrix-core projections (large batches only: the small-batch
// kernels read the fp32 reductors), or an undefined tensor
Tensor reductors_split(const Tensor& red, int A) {
    if (A < 2049) return Tensor();
    const int ne = (int)red.size(0), R = (int)red.size(1), d = (int)red.size(2);
    const size_t nbytes = qmll_reductor_presplit_bytes(ne, R, d);
    if (nbytes == 0) return Tensor();
    return prepared_form(red, 1, [&](const Tensor& u) {
        Tensor out = at::empty({(int64_t)nbytes}, u.options().dtype(at::kByte));
        check(qmll_reductor_presplit(fp(u), ne, R, d, out.data_ptr(), nbytes, stream()), "qmll_reductor_presplit");
        return out;
    });
}
const void* vp(const Tensor& t) { return t.defined() && t.numel() ? t.const_data_ptr() : nullptr; }

Tensor project_typed_impl(const Tensor& rep, const Tensor& sorted_slots, const Tensor& type_offsets,
                          const Tensor& reductors) {
    Tensor r = f32(rep), red = f32(reductors), ss = i32(sorted_slots), off = i32(type_offsets);
    need_cuda(r, "rep");
    const int ne = (int)red.size(0), R = (int)red.size(1), d = (int)red.size(2), A = (int)ss.size(0);
    TORCH_CHECK(r.dim() == 2 && r.size(1) == R && off.size(0) == ne + 1,
                "project_typed: rep, reductors and offsets do not fit together");
    Tensor x = at::empty({A, d}, r.options());
    Tensor split = reductors_split(red, A);
    check(qmll_project_typed(fp(r), ip(ss), ip(off), fp(red), vp(split), A, ne, R, d, A ? x.data_ptr<float>() : nullptr,
                             stream()),
          "qmll_project_typed");
    return x;
}

Tensor project_typed_backward(const Tensor& gx, const Tensor& sorted_slots, const Tensor& type_offsets,
                              const Tensor& reductors, const Tensor& types, int64_t nslots) {
    Tensor g = f32(gx), red = f32(reductors), ss = i32(sorted_slots), off = i32(type_offsets);
    Tensor ty = i32(types).reshape({-1});
    need_cuda(g, "gx");
    const int ne = (int)red.size(0), R = (int)red.size(1), d = (int)red.size(2), A = (int)ss.size(0), N = (int)nslots;
    TORCH_CHECK(g.size(0) == A && g.size(1) == d && ty.size(0) == N, "project_typed_backward: gx does not fit ", A,
                " atoms, d=", d);
    // every slot a real atom: the kernel writes every row of a known element and zeroes the rest
    const bool full = A == N;
    Tensor g_rep = full ? at::empty({N, R}, g.options()) : at::zeros({N, R}, g.options());
    Tensor split = reductors_split(red, A);
    check(qmll_project_typed_backward(fp(g), ip(ss), ip(off), fp(red), vp(split), full ? ip(ty) : nullptr, A, N, ne, R, d,
                                      N ? g_rep.data_ptr<float>() : nullptr, stream()),
          "qmll_project_typed_backward");
    return g_rep;
}

struct ProjectFn : public Function<ProjectFn> {
    static Tensor forward(AutogradContext* ctx, const Tensor& rep, const Tensor& ss, const Tensor& off, const Tensor& red,
                          const Tensor& types) {
        ctx->save_for_backward({ss, off, red, types});
        ctx->saved_data["nslots"] = rep.size(0);
        return project_typed_impl(rep, ss, off, red);
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        const variable_list s = ctx->get_saved_variables();
        variable_list out(5);
        if (grads[0].defined())
            out[0] = project_typed_backward(grads[0].contiguous(), s[0], s[1], s[2], s[3], ctx->saved_data["nslots"].toInt());
        return out;
    }
};

Tensor project_typed(const Tensor& rep, const Tensor& ss, const Tensor& off, const Tensor& red, const Tensor& types) {
    return ProjectFn::apply(rep, ss, off, red, types);
}

// the fused SORF kernel on rows x f32 [A,d] of a model (ne elements): shape checks of the model's tensors and the launch;
// e f32 [nslots] zero-filled, gx f32 [A,d] or nullptr
void sorf_energy_sorted_raw(const float* x, const int* off, const int* ss, int A, int d_x, int ne_off, const Tensor& Dmat,
                            const Tensor& bias, const Tensor& alpha, const Tensor& cn, const Tensor& nt, float* e, float* gx) {
    Tensor DD = f32(Dmat), bb = f32(bias), al = alpha32(alpha);
    need_cuda(DD, "Dmat");
    TORCH_CHECK(DD.dim() == 4, "sorf_energy_sorted: Dmat is [", DD.sizes(), "], expected [elements, transforms, stacks, d]");
    const int ne = (int)DD.size(0), Tn = (int)DD.size(1), S = (int)DD.size(2), d = (int)DD.size(3);
    const int T = nt.item<int>();
    TORCH_CHECK(d_x == d && ne_off == ne, "sorf_energy_sorted: x has ", d_x, " columns and the offsets ", ne_off,
                " elements, expected ", d, " and ", ne);
    TORCH_CHECK(T == Tn, "sorf_energy_sorted: ", Tn, " diagonals stored per stack, ", T, " transforms asked for");
    TORCH_CHECK(bb.dim() == 2 && bb.size(0) == ne && bb.size(1) == (int64_t)S * d && al.numel() == (int64_t)S * d,
                "sorf_energy_sorted: bias [", bb.sizes(), "] / alpha with ", al.numel(), " entries do not fit ", ne,
                " elements and ", S * d, " features");
    // the largest |bias|, a constant of the model: computed once per tensor version, kept on the device
    Tensor bmax = prepared_form(bb, 2, [](const Tensor& b) { return b.abs().max().reshape({1}); });
    check(qmll_sorf_energy_sorted(x, off, ss, fp(DD), fp(bb), fp(al), fp(bmax), A, ne, d, S, T, scalar(cn), e, A ? gx : nullptr,
                                  stream()),
          "qmll_sorf_energy_sorted");
}

// e_zeroed: the caller's zero-filled f32 [nslots] for the energies (one fill then serves several outputs), or undefined
std::tuple<Tensor, Tensor> sorf_energy_sorted_impl(const Tensor& x_, const Tensor& type_offsets, const Tensor& sorted_slots,
                                                   const Tensor& Dmat, const Tensor& bias, const Tensor& alpha,
                                                   const Tensor& cn, const Tensor& nt, int64_t nslots, bool with_grad,
                                                   const Tensor& e_zeroed = Tensor()) {
    Tensor x = f32(x_), off = i32(type_offsets), ss = i32(sorted_slots);
    need_cuda(x, "x");
    const int A = (int)ss.size(0);
    TORCH_CHECK(x.dim() == 2 && x.size(0) == A && off.dim() == 1, "sorf_energy_sorted: x is [", x.sizes(), "] for ", A, " atoms");
    Tensor e = e_zeroed.defined() ? e_zeroed : at::zeros({nslots}, x.options());
    Tensor gx = with_grad ? at::empty({A, x.size(1)}, x.options()) : empty_like_none(x);
    sorf_energy_sorted_raw(fp(x), ip(off), ip(ss), A, (int)x.size(1), (int)off.size(0) - 1, Dmat, bias, alpha, cn, nt,
                           nslots ? e.data_ptr<float>() : nullptr, with_grad ? gx.data_ptr<float>() : nullptr);
    return {e, gx};
}

// backward shared by the two element-sorted energy operators: gradient rows times the energy
// gradient of each row's slot
variable_list sorted_backward(AutogradContext* ctx, const variable_list& grads, size_t ninputs, const char* who) {
    variable_list out(ninputs);
    if (!grads[0].defined()) return out;
    const variable_list s = ctx->get_saved_variables();
    const Tensor gx = s[0], ss = s[1];
    TORCH_CHECK(!(gx.numel() == 0 && ss.numel() != 0), who,
                " was called with with_grad=False but a gradient is requested");
    out[0] = gx * grads[0].index_select(0, ss.to(at::kLong)).unsqueeze(1);
    return out;
}

struct SorfEnergySortedFn : public Function<SorfEnergySortedFn> {
    static variable_list forward(AutogradContext* ctx, const Tensor& x, const Tensor& off, const Tensor& ss,
                                 const Tensor& Dmat, const Tensor& bias, const Tensor& alpha, const Tensor& cn,
                                 const Tensor& nt, int64_t nslots, bool with_grad) {
        auto r = sorf_energy_sorted_impl(x, off, ss, Dmat, bias, alpha, cn, nt, nslots, with_grad);
        ctx->save_for_backward({std::get<1>(r), ss});
        ctx->mark_non_differentiable({std::get<1>(r)});
        ctx->set_materialize_grads(false);
        return {std::get<0>(r), std::get<1>(r)};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        return sorted_backward(ctx, grads, 10, "sorf_energy_sorted");
    }
};

std::tuple<Tensor, Tensor> sorf_energy_sorted(const Tensor& x, const Tensor& off, const Tensor& ss, const Tensor& Dmat,
                                              const Tensor& bias, const Tensor& alpha, const Tensor& cn, const Tensor& nt,
                                              int64_t nslots, bool with_grad) {
    auto r = SorfEnergySortedFn::apply(x, off, ss, Dmat, bias, alpha, cn, nt, nslots, with_grad);
    return {r[0], r[1]};
}

// the fused RFF kernel on rows x f32 [A,d]: shape checks of the model's tensors and the launch (e zero-filled)
void rff_energy_sorted_raw(const float* x, const int* off, const int* ss, int A, int d_x, int ne_off, const Tensor& W,
                           const Tensor& b, const Tensor& alpha, float* e, float* gx) {
    Tensor WW = f32(W), bb = f32(b), al = alpha32(alpha);
    need_cuda(WW, "W");
    TORCH_CHECK(WW.dim() == 3 && bb.dim() == 2, "rff_energy_sorted: W is [", WW.sizes(), "], b is [", bb.sizes(), "]");
    const int ne = (int)WW.size(0), d = (int)WW.size(1), F = (int)WW.size(2);
    TORCH_CHECK(d_x == d && ne_off == ne && bb.size(0) == ne && bb.size(1) == F,
                "rff_energy_sorted: x, W and b do not fit together");
    TORCH_CHECK(al.numel() == F, "rff_energy_sorted: alpha has ", al.numel(), " entries for ", F, " features");
    Tensor Wsplit = prepared_form(WW, 0, [&](const Tensor& w) {
        const size_t nbytes = qmll_rff_presplit_bytes(ne, d, F);
        TORCH_CHECK(nbytes > 0, "rff_energy_sorted: the fused kernel exists for 64 or 128 components and a multiple of 32 "
                    "features, not ", d, " and ", F);
        Tensor out = at::empty({(int64_t)nbytes}, w.options().dtype(at::kByte));
        check(qmll_rff_presplit(fp(w), ne, d, F, out.data_ptr(), nbytes, stream()), "qmll_rff_presplit");
        return out;
    });
    check(qmll_rff_energy_sorted(x, off, ss, Wsplit.const_data_ptr(), fp(bb), fp(al), A, ne, d, F, e, A ? gx : nullptr, stream()),
          "qmll_rff_energy_sorted");
}

std::tuple<Tensor, Tensor> rff_energy_sorted_impl(const Tensor& x_, const Tensor& type_offsets, const Tensor& sorted_slots,
                                                  const Tensor& W, const Tensor& b, const Tensor& alpha, int64_t nslots,
                                                  bool with_grad, const Tensor& e_zeroed = Tensor()) {
    Tensor x = f32(x_), off = i32(type_offsets), ss = i32(sorted_slots);
    need_cuda(x, "x");
    const int A = (int)ss.size(0);
    TORCH_CHECK(x.dim() == 2 && x.size(0) == A && off.dim() == 1, "rff_energy_sorted: x is [", x.sizes(), "] for ", A, " atoms");
    Tensor e = e_zeroed.defined() ? e_zeroed : at::zeros({nslots}, x.options());
    Tensor gx = with_grad ? at::empty({A, x.size(1)}, x.options()) : empty_like_none(x);
    rff_energy_sorted_raw(fp(x), ip(off), ip(ss), A, (int)x.size(1), (int)off.size(0) - 1, W, b, alpha,
                          nslots ? e.data_ptr<float>() : nullptr, with_grad ? gx.data_ptr<float>() : nullptr);
    return {e, gx};
}


struct RffEnergySortedFn : public Function<RffEnergySortedFn> {
    static variable_list forward(AutogradContext* ctx, const Tensor& x, const Tensor& off, const Tensor& ss,
                                 const Tensor& W, const Tensor& b, const Tensor& alpha, int64_t nslots, bool with_grad) {
        auto r = rff_energy_sorted_impl(x, off, ss, W, b, alpha, nslots, with_grad);
        ctx->save_for_backward({std::get<1>(r), ss});
        ctx->mark_non_differentiable({std::get<1>(r)});
        ctx->set_materialize_grads(false);
        return {std::get<0>(r), std::get<1>(r)};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        return sorted_backward(ctx, grads, 8, "rff_energy_sorted");
    }
};

std::tuple<Tensor, Tensor> rff_energy_sorted(const Tensor& x, const Tensor& off, const Tensor& ss, const Tensor& W,
                                             const Tensor& b, const Tensor& alpha, int64_t nslots, bool with_grad) {
    auto r = RffEnergySortedFn::apply(x, off, ss, W, b, alpha, nslots, with_grad);
    return {r[0], r[1]};
}

// ---- the whole fused predict chain as one operator ---------------------------------------
// energies [B] of forward(X, Z, atomIDs, molIDs, atom_counts) (models/hadamard_features.py:82-123):
// representation, sort by element, projection, SORF + cos + energy, and -- when the coordinates
// require a gradient -- the backward chain as well (the fused kernel returns dE/dx itself, the
// projection transpose and the representation VJP follow), saved for one autograd node.  One
// dispatch and one node instead of five of each: what a TorchScript caller that evaluates a single
// molecule per step pays for is dispatch, not kernels.
#define MODEL_TENSORS                                                                                   \
    const Tensor &reductors, const Tensor &Dmat, const Tensor &bias, const Tensor &alpha, const Tensor &cn, \
        const Tensor &nt, const Tensor &model_species

// rff = true: `Dmat` holds W [ne,d,F], `bias` holds b [ne,F]; cn and nt are unused.
// model_species: the charges of the model's own elements in the order of its reductors / Dmat /
// bias rows (the reference selects each element's atoms with Z == e over the MODEL's elements,
// models/hadamard_features.py:99-107, while the representation indexes its bins by the
// REPRESENTATION's species); an empty tensor says the two lists are the same.
// gscale: factor on the returned coordinate gradient (-1: forces)
Tensor fchl_sorf_energy_impl(FCHL_TENSORS, MODEL_TENSORS, bool with_grad, Tensor* gX_out, bool rff = false,
                             float gscale = 1.0f) {
    FchlInputs in = prepare(FCHL_PASS, false);
    need_cuda(reductors, "reductors");
    TORCH_CHECK(reductors.dim() == 3 && reductors.size(1) == in.R, "fchl_sorf_energy: reductors are [",
                reductors.sizes(), "], the representation has ", in.R, " entries per atom");
    const int ne = (int)reductors.size(0), R = in.R, d = (int)reductors.size(2), A = in.A, B = in.B, n = in.n;
    const bool own_list = model_species.numel() != 0;
    if (!own_list) {
        TORCH_CHECK(ne == in.prm.nspecies, "fchl_sorf_energy: the model has ", ne, " elements, the representation ",
                    in.prm.nspecies, " species, and no model species were given");
    } else {
        TORCH_CHECK(model_species.numel() == ne, "fchl_sorf_energy: ", model_species.numel(), " model species for ", ne,
                    " reductors");
        need_cuda(model_species, "model_species");
    }
    Tensor Zb = f32(Z.dim() == 1 ? Z.unsqueeze(0) : Z), sp = f32(species), msp = own_list ? f32(model_species) : Tensor();
    Tensor red = f32(reductors);
    TORCH_CHECK(Zb.dim() == 2 && Zb.size(0) == B && Zb.size(1) == n, "fchl_sorf_energy: charges are [", Zb.sizes(),
                "], coordinates [", in.X.sizes(), "]");
    const int64_t nslots = (int64_t)B * n;
    // few allocations, cut up by hand: for one molecule the step is as long as its host side
    //   ints:    element index by the representation's list | by the model's (only when it has its own) |
    //            sorted slots | offsets | workspace of the sort
    //   out:     per-slot energies | dE/dX   (what must start at zero)
    //   scratch: representation | projected rows | their gradient | gradient of the representation
    const size_t sort_bytes = qmll_sort_atoms_workspace(A, ne);
    const int64_t types_ints = nslots * (own_list ? 2 : 1);
    Tensor ints = at::empty({types_ints + A + ne + 1 + (int64_t)(sort_bytes / 4) + 1}, in.X.options().dtype(at::kInt));
    int* types = ints.data_ptr<int>();
    int* sort_types = own_list ? types + nslots : types;
    int* ss = types + types_ints;
    int* off = ss + A;
    int* sort_work = off + ne + 1;
    const int64_t nzero = (with_grad ? 4 : 1) * nslots;
    Tensor out = at::empty({nzero}, in.X.options());
    float* e_slots = nzero ? out.data_ptr<float>() : nullptr;
    check(qmll_prepare_batch(fp(Zb), ip(in.natoms), fp(sp), in.prm.nspecies, fp(msp), ne, ip(in.atomIDs), ip(in.molIDs), B, n,
                             A, sort_work, sort_bytes, types, own_list ? sort_types : nullptr, ss, off, e_slots,
                             (size_t)nzero, stream()),
          "qmll_prepare_batch");
    auto pad = [](int64_t v) { return (v + 63) / 64 * 64; };          // every part 256-byte aligned
    const int64_t rep_n = pad(nslots * R), x_n = pad((int64_t)A * d);
    Tensor scratch = at::empty({rep_n + x_n + (with_grad ? x_n + rep_n : 0) + 64}, in.X.options());
    float* rep = scratch.data_ptr<float>();
    float* x = rep + rep_n;
    float* gx = with_grad ? x + x_n : nullptr;
    float* g_rep = with_grad ? gx + x_n : nullptr;
    // the forward kernel writes every bin of a listed atom's row, and only the rows of listed
    // atoms are read below, so the padded rows need no clearing
    check(qmll_fchl19_forward(FCHL_ABI_T(in, types), rep, stream()), "qmll_fchl19_forward");
    Tensor split = reductors_split(red, A);
    check(qmll_project_typed(rep, ss, off, fp(red), vp(split), A, ne, R, d, x, stream()), "qmll_project_typed");
    if (rff)
        rff_energy_sorted_raw(x, off, ss, A, d, ne, Dmat, bias, alpha, e_slots, gx);
    else
        sorf_energy_sorted_raw(x, off, ss, A, d, ne, Dmat, bias, alpha, cn, nt, e_slots, gx);
    Tensor energies = at::empty({B}, in.X.options());
    if (!with_grad) {        // the sums alone (A = 0), by the kernel that sums them beside the backward projection
        check(qmll_project_typed_backward_sums(nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, ne, R, d, nullptr,
                                               e_slots, B, n, B ? energies.data_ptr<float>() : nullptr, stream()),
              "qmll_project_typed_backward_sums");
        return energies;
    }
    // rows of listed atoms whose element the model does not hold are zeroed (sort_types); the rows of
    // padded slots are never read by the kernel below
    check(qmll_project_typed_backward_sums(gx, ss, off, fp(red), vp(split), sort_types, A, (int)nslots, ne, R, d, g_rep,
                                           e_slots, B, n, B ? energies.data_ptr<float>() : nullptr, stream()),
          "qmll_project_typed_backward_sums");
    Tensor gX = out.narrow(0, nslots, 3 * nslots).view({B, n, 3});
    check(qmll_fchl19_vjp_scaled(FCHL_ABI_T(in, types), g_rep, gscale, nslots ? gX.data_ptr<float>() : nullptr, stream()),
          "qmll_fchl19_vjp");
    *gX_out = gX;
    return energies;
}

struct FchlSorfEnergyFn : public Function<FchlSorfEnergyFn> {
    static variable_list forward(AutogradContext* ctx, FCHL_TENSORS, MODEL_TENSORS, bool with_grad) {
        Tensor gX;
        Tensor e = fchl_sorf_energy_impl(FCHL_PASS, reductors, Dmat, bias, alpha, cn, nt, model_species, with_grad, &gX);
        if (!with_grad) gX = empty_like_none(e);
        ctx->save_for_backward({gX});
        ctx->mark_non_differentiable({gX});
        ctx->set_materialize_grads(false);
        ctx->saved_data["xdim"] = X.dim();
        return {e, gX};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        variable_list out(24);
        if (!grads[0].defined()) return out;
        const Tensor gX = ctx->get_saved_variables()[0];                 // [B,n,3], dE_m/dX of each molecule
        TORCH_CHECK(gX.dim() == 3, "fchl_sorf_energy was called with with_grad=False but a gradient is requested");
        Tensor g = gX * grads[0].reshape({-1, 1, 1});
        out[0] = ctx->saved_data["xdim"].toInt() == 2 ? g.squeeze(0) : g;
        return out;
    }
};

// returns (energies [B], dE/dX [B,n,3] or an empty tensor when with_grad is false)
std::tuple<Tensor, Tensor> fchl_sorf_energy(FCHL_TENSORS, MODEL_TENSORS, bool with_grad) {
    auto r = FchlSorfEnergyFn::apply(FCHL_PASS, reductors, Dmat, bias, alpha, cn, nt, model_species, with_grad);
    return {r[0], r[1]};
}

// (energies [B], forces [B,n,3] = -dE/dX) outside autograd: what a predict call wants, the sign applied
// inside the last kernel of the chain instead of by an elementwise pass afterwards
void no_graph(const Tensor& X, const char* who) {
    TORCH_CHECK(!(at::GradMode::is_enabled() && X.requires_grad()), who,
                " builds no autograd graph: call it under no_grad, or use the _energy operator for a differentiable result");
}
std::tuple<Tensor, Tensor> fchl_sorf_forces(FCHL_TENSORS, MODEL_TENSORS) {
    no_graph(X, "fchl_sorf_forces");
    at::NoGradGuard guard;
    Tensor F;
    Tensor e = fchl_sorf_energy_impl(FCHL_PASS, reductors, Dmat, bias, alpha, cn, nt, model_species, true, &F, false, -1.0f);
    return {e, X.dim() == 2 ? F.squeeze(0) : F};
}
std::tuple<Tensor, Tensor> fchl_rff_forces(FCHL_TENSORS, const Tensor& reductors, const Tensor& W, const Tensor& b,
                                           const Tensor& alpha, const Tensor& model_species) {
    no_graph(X, "fchl_rff_forces");
    at::NoGradGuard guard;
    Tensor F;
    Tensor e = fchl_sorf_energy_impl(FCHL_PASS, reductors, W, b, alpha, Tensor(), Tensor(), model_species, true, &F, true,
                                     -1.0f);
    return {e, X.dim() == 2 ? F.squeeze(0) : F};
}

// the same chain with random Fourier features (models/random_features.py:82-102)
struct FchlRffEnergyFn : public Function<FchlRffEnergyFn> {
    static variable_list forward(AutogradContext* ctx, FCHL_TENSORS, const Tensor& reductors, const Tensor& W,
                                 const Tensor& b, const Tensor& alpha, const Tensor& model_species, bool with_grad) {
        Tensor gX;
        Tensor e = fchl_sorf_energy_impl(FCHL_PASS, reductors, W, b, alpha, Tensor(), Tensor(), model_species, with_grad,
                                         &gX, true);
        if (!with_grad) gX = empty_like_none(e);
        ctx->save_for_backward({gX});
        ctx->mark_non_differentiable({gX});
        ctx->set_materialize_grads(false);
        ctx->saved_data["xdim"] = X.dim();
        return {e, gX};
    }
    static variable_list backward(AutogradContext* ctx, variable_list grads) {
        variable_list out(22);
        if (!grads[0].defined()) return out;
        const Tensor gX = ctx->get_saved_variables()[0];
        TORCH_CHECK(gX.dim() == 3, "fchl_rff_energy was called with with_grad=False but a gradient is requested");
        Tensor g = gX * grads[0].reshape({-1, 1, 1});
        out[0] = ctx->saved_data["xdim"].toInt() == 2 ? g.squeeze(0) : g;
        return out;
    }
};

std::tuple<Tensor, Tensor> fchl_rff_energy(FCHL_TENSORS, const Tensor& reductors, const Tensor& W, const Tensor& b,
                                           const Tensor& alpha, const Tensor& model_species, bool with_grad) {
    auto r = FchlRffEnergyFn::apply(FCHL_PASS, reductors, W, b, alpha, model_species, with_grad);
    return {r[0], r[1]};
}

}  // namespace

// operator names and argument order of the reference (torchscript/FCHL19.cpp:318-333)
TORCH_LIBRARY(qml_lightning_fchl, m) {
    m.def("fchl_forwards", &fchl_forwards);
    m.def("fchl_backwards", &fchl_backwards);
    m.def("get_fchl_and_derivative", &get_fchl_and_derivative);
    m.def("get_element_types", &element_types);
    m.def("get_num_neighbours", &get_num_neighbours);
    m.def("get_neighbour_list", &get_neighbour_list);
}

// torchscript/SORF.cpp:138-150, plus the fused predict operators
TORCH_LIBRARY(qml_lightning_sorf, m) {
    m.def("get_SORF_coefficients", &get_SORF_coefficients);
    m.def("get_SORF_coefficients_backward", &sorf_coefficients_backward);
    m.def("get_cos_features", &get_cos_features);
    m.def("get_cos_features_backward", &cos_features_backward);
    m.def("sorf_energy", &sorf_energy);
    m.def("sorf_energy_typed", &sorf_energy_typed);
    m.def("sort_by_type", &sort_by_type);
    m.def("project_typed", &project_typed);
    m.def("project_typed_backward", &project_typed_backward);
    m.def("sorf_energy_sorted", &sorf_energy_sorted);
    m.def("rff_energy_sorted", &rff_energy_sorted);
    m.def("fchl_sorf_energy", &fchl_sorf_energy);
    m.def("fchl_rff_energy", &fchl_rff_energy);
    m.def("fchl_sorf_forces", &fchl_sorf_forces);
    m.def("fchl_rff_forces", &fchl_rff_forces);
}

// names the loader can test for
extern "C" int qmll_torch_ops_version(void) { return 1; }
