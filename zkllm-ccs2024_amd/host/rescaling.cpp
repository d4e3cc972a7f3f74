#include "rescaling.hpp"

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

Rescaling::Rescaling(uint scaling_factor) : scaling_factor(scaling_factor), tl_rem(-static_cast<int>(scaling_factor >> 1), scaling_factor), rem_tensor_ptr(nullptr) {}

FrTensor Rescaling::operator()(const FrTensor& X) {
    if (rem_tensor_ptr) delete rem_tensor_ptr;
    rem_tensor_ptr = new FrTensor(X.size);
    FrTensor out(X.size);
    ZKC(zk_rescale(out.gpu_data, rem_tensor_ptr->gpu_data, X.gpu_data, scaling_factor, X.size, nullptr));
    return out;
}
Rescaling::~Rescaling() { if (rem_tensor_ptr) delete rem_tensor_ptr; }

// rescaling.cu:41-79.  Challenge order: u, v, (alpha, beta).
vector<Claim> Rescaling::prove(const FrTensor& X, const FrTensor& X_) {
    if (X.size != X_.size) throw std::runtime_error("Error: the size of X and X_ should be the same.");
    if (!rem_tensor_ptr) throw std::runtime_error("Rescaling::prove called before operator()");
    auto u = random_vec(ceilLog2(X.size));
    auto v = random_vec(ceilLog2(X.size));
    auto rand_temp = random_vec(2);
    vector<Polynomial> proof;

    auto rem = rem_tensor_ptr->pad({rem_tensor_ptr->size});
    auto m = tl_rem.prep(rem);
    const Fr_t lhs = X(u);
    zk_record(lhs);
    if (lhs != X_(u) * Fr_t({scaling_factor, 0, 0, 0, 0, 0, 0, 0}) + rem(u)) throw std::runtime_error("Error: the rem is not correct.");
    tl_rem.prove(rem, m, rand_temp[0], rand_temp[1], u, v, proof);
    cout << "Rescaling proof complete." << endl;
    return {};
}
