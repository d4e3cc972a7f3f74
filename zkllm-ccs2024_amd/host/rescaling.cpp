#include "rescaling.hpp"

#include <cstdlib>

#include "../../include/zkllm_hip.h"

#define ZKC(call) zk_check((call), #call)

Rescaling::Rescaling(uint scaling_factor) : scaling_factor(scaling_factor), tl_rem(-static_cast<int>(scaling_factor >> 1), scaling_factor), rem_tensor_ptr(nullptr) {}

FrTensor Rescaling::operator()(const FrTensor& X) { return rescale(X, out_ints_lazy); }
FrTensor Rescaling::rescale(const FrTensor& X, bool ints_out) {
    rem_hold = std::make_shared<FrTensor>(X.size);
    rem_tensor_ptr = rem_hold.get();
    FrTensor out(X.size);
    // the remainders are written as int32 as well: the range proof's index pass, evaluation and first round read that form
    // the rescaled values too, when they fit (activations do): lookups, products and evaluations downstream read that form
    // (asked for by the caller: whether they fit is read back, a host round trip that a block which shares the device with
    // the openings' kernels pays with milliseconds)
    // lean: the field elements of the remainders are written only where something reads them
    // (the same condition under which prove_begin pads the int32 form alone and the lookup job reads nothing else)
    const bool ints_only = lean && zk_lookup_ints_suffice((size_t)1 << ceilLog2(X.size), tl_rem.table.size);
    void* rem_fr = ints_only ? nullptr : rem_tensor_ptr->gpu_data;
    if (ints_out && out_ints_lazy) {
        void* flag = nullptr;
        void* oi = out.ints_for_producer_unchecked(&flag);
        ZKC(zk_rescale_ints_both_flag(out.gpu_data, oi, flag, rem_fr, rem_hold->ints_for_producer(), X.gpu_data, scaling_factor, X.size, nullptr));
    } else if (ints_out) {
        int fits = 0;
        ZKC(zk_rescale_ints_both(out.gpu_data, out.ints_for_producer(), &fits, rem_fr, rem_hold->ints_for_producer(), X.gpu_data, scaling_factor, X.size, nullptr));
        if (!fits) out.drop_kept();
    } else ZKC(zk_rescale_ints(out.gpu_data, rem_fr, rem_hold->ints_for_producer(), X.gpu_data, scaling_factor, X.size, nullptr));
    return out;
}
Rescaling::~Rescaling() {}

// rescaling.cu:41-79.  Challenge order: u, v, (alpha, beta).
vector<Claim> Rescaling::prove(const FrTensor& X, const FrTensor& X_) {
    Pending p = prove_begin(X, X_);
    prove_end(p);
    return {};
}
Rescaling::Challenges Rescaling::draw(uint size) {
    Challenges ch;
    ch.u = random_vec(ceilLog2(size));
    ch.v = random_vec(ceilLog2(size));
    ch.rand_temp = random_vec(2);
    return ch;
}
Rescaling::Pending Rescaling::prove_begin(const FrTensor& X, const FrTensor& X_) {
    if (X.size != X_.size) throw std::runtime_error("Error: the size of X and X_ should be the same.");
    if (!rem_tensor_ptr) throw std::runtime_error("Rescaling::prove called before operator()");
    return prove_begin(X, X_, draw(X.size));
}
Rescaling::Pending Rescaling::prove_begin(const FrTensor& X, const FrTensor& X_, const Challenges& ch) {
    if (X.size != X_.size) throw std::runtime_error("Error: the size of X and X_ should be the same.");
    if (!rem_tensor_ptr) throw std::runtime_error("Rescaling::prove called before operator()");
    const vector<Fr_t>&u = ch.u, &v = ch.v, &rand_temp = ch.rand_temp;
    if (u.size() != ceilLog2(X.size) || v.size() != u.size() || rand_temp.size() != 2) throw std::runtime_error("Rescaling::prove: challenges do not match the shape");

    Pending p;
    if (rem_tensor_ptr->size == (1u << ceilLog2(rem_tensor_ptr->size))) p.rem = rem_hold;
    else {
        // with an int32 form that a job of this size reads alone, the padded field elements are never read: not written
        const uint padded_size = 1u << ceilLog2(rem_tensor_ptr->size);
        const bool ints_only = rem_tensor_ptr->kept_ints() && zk_lookup_ints_suffice(padded_size, tl_rem.table.size);
        auto padded = ints_only ? std::make_shared<FrTensor>(padded_size) : std::make_shared<FrTensor>(rem_tensor_ptr->pad({rem_tensor_ptr->size}));
        if (const void* h = rem_tensor_ptr->kept_ints()) {          // the int32 form is padded with the same zeros
            char* dst = (char*)padded->ints_for_producer();
            const size_t have = sizeof(int32_t) * (size_t)rem_tensor_ptr->size, all = sizeof(int32_t) * (size_t)padded->size;
            ZKC(zk_memcpy_d2d(dst, zk_fr_fold_prepared_ints(h), have, nullptr));
            ZKC(zk_memset(dst + have, 0, all - have, nullptr));
        }
        p.rem = padded;
    }
    p.m.reset(new FrTensor(tl_rem.prep(*p.rem)));
    // X_(u) and rem(u) in one pass over the two tensors (the padding of the remainders is zeros: the unpadded tensor has the same
    // extension and the others' length).  X = scaling_factor X_ + rem element by element, so X(u) is that combination of the two
    // values: X itself, 32 bytes an element, is read only with ZKLLM_CHECK_CLAIMS=1, which evaluates it and compares as
    // rescaling.cu:52-57 does.
    const char* check_env = getenv("ZKLLM_CHECK_CLAIMS");
    const bool read_X = check_env && check_env[0] == '1';
    vector<Fr_t> ev = read_X ? FrTensor::me_batch({&X_, rem_tensor_ptr, &X}, u) : FrTensor::me_batch({&X_, rem_tensor_ptr}, u);
    p.lhs = ev[0] * Fr_t({scaling_factor, 0, 0, 0, 0, 0, 0, 0}) + ev[1];
    if (read_X && p.lhs != ev[2]) throw std::runtime_error("Error: the rem is not correct.");
    p.look = tl_rem.prove_begin(*p.rem, *p.m, rand_temp[0], rand_temp[1], u, v);
    return p;
}
void Rescaling::prove_end(Pending& p) {
    zk_record(p.lhs);
    tLookup::prove_end(p.look);
    cout << "Rescaling proof complete." << endl;
}
