#include "zkrelu.hpp"

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

zkReLU::zkReLU(uint scaling_factor)
    : scaling_factor(scaling_factor), tl_rem(-static_cast<int>(scaling_factor >> 1), scaling_factor),
      sign_tensor_ptr(nullptr), abs_tensor_ptr(nullptr), rem_tensor_ptr(nullptr), m_tensor_ptr(nullptr) {}

// zkrelu.cu:31-39
FrTensor zkReLU::decomp(const FrTensor& X, FrTensor& sign, FrTensor& abs, FrTensor& rem) {
    if (sign.size != X.size || abs.size != X.size || rem.size != X.size) throw std::runtime_error("Incompatible dimensions");
    FrTensor res(X.size);
    ZKC(zk_relu_decomp(res.gpu_data, sign.gpu_data, abs.gpu_data, rem.gpu_data, X.gpu_data, scaling_factor, X.size, nullptr));
    return res;
}

// zkrelu.cu:41-54
FrTensor zkReLU::operator()(const FrTensor& X) {
    delete sign_tensor_ptr; sign_tensor_ptr = nullptr;
    delete abs_tensor_ptr;  abs_tensor_ptr = nullptr;
    delete rem_tensor_ptr;  rem_tensor_ptr = nullptr;
    delete m_tensor_ptr;    m_tensor_ptr = nullptr;
    sign_tensor_ptr = new FrTensor(X.size);
    abs_tensor_ptr = new FrTensor(X.size);
    rem_tensor_ptr = new FrTensor(X.size);
    FrTensor res = decomp(X, *sign_tensor_ptr, *abs_tensor_ptr, *rem_tensor_ptr);
    m_tensor_ptr = new FrTensor(tl_rem.prep(*rem_tensor_ptr));
    return res;
}

void zkReLU::prove(const FrTensor&, const FrTensor&) {}

zkReLU::~zkReLU() {
    delete sign_tensor_ptr;
    delete abs_tensor_ptr;
    delete rem_tensor_ptr;
    delete m_tensor_ptr;
}
