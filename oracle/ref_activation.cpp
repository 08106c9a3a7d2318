// C entry points over the reference's own activation registry (include/Activation.h:403-438),
// compiled from the reference sources where they lie; test infrastructure only.
#include "Activation.h"

#include <cstddef>

namespace {
const char* kNames[] = { "leaky", "linear", "loggy", "logistic", "mish", "relu", "softplus", "swish", "tanh" };
}

extern "C" {

// type follows include/ActivationTypes.h:19-30
int ref_activate(int type, float* x, std::size_t n)
{
    if (type < 0 || type > 8) return 1;
    auto act = px::Activations<>::get(kNames[type]);
    act->apply(x, x + n);
    return 0;
}

int ref_gradient(int type, const float* x, std::size_t n, float* delta)
{
    if (type < 0 || type > 8) return 1;
    auto act = px::Activations<>::get(kNames[type]);
    act->gradient(delta, delta + n, x);
    return 0;
}

}
