// A host without Python: loads the operator library, a TorchScript model file and the input
// tensors written next to it, runs forward + backward on the GPU and prints the energies
// and forces.  Used by tests/test_gpu_model.py to show that a saved model needs nothing but
// libtorch, libqmll_torch.so and libqmll.so.
//
//   run_scripted <libqmll_torch.so> <model.pt> <inputs.pt>
//
// inputs.pt is a scripted module whose attributes X, Z, atomIDs, molIDs, atom_counts hold
// the batch (the portable way to hand tensors to libtorch).
#include <dlfcn.h>
#include <torch/script.h>

#include <cstdio>
#include <iostream>

int main(int argc, char** argv) {
    if (argc != 4) {
        std::fprintf(stderr, "usage: %s <libqmll_torch.so> <model.pt> <inputs.pt>\n", argv[0]);
        return 2;
    }
    if (!dlopen(argv[1], RTLD_NOW | RTLD_GLOBAL)) {
        std::fprintf(stderr, "cannot load %s: %s\n", argv[1], dlerror());
        return 3;
    }
    try {
        torch::jit::script::Module model = torch::jit::load(argv[2], torch::kCUDA);
        torch::jit::script::Module in = torch::jit::load(argv[3], torch::kCUDA);
        at::Tensor X = in.attr("X").toTensor().clone().set_requires_grad(true);
        std::vector<torch::jit::IValue> args{X, in.attr("Z").toTensor(), in.attr("atomIDs").toTensor(),
                                             in.attr("molIDs").toTensor(), in.attr("atom_counts").toTensor()};
        at::Tensor E = model.forward(args).toTensor();
        (-E.sum()).backward();
        at::Tensor F = X.grad().cpu().contiguous(), Ec = E.detach().cpu().contiguous();
        std::printf("energies %ld\n", (long)Ec.numel());
        for (int64_t i = 0; i < Ec.numel(); ++i) std::printf("%.9g\n", (double)Ec.data_ptr<float>()[i]);
        std::printf("forces %ld\n", (long)F.numel());
        for (int64_t i = 0; i < F.numel(); ++i) std::printf("%.9g\n", (double)F.data_ptr<float>()[i]);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "error: %s\n", e.what());
        return 1;
    }
    return 0;
}
