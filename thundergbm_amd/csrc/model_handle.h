// The model handle of the C ABI (`Tree*&` in the reference's scikit_tgbm.cpp): all trees, iteration-major, the
// class trees of an iteration next to each other. Opaque to callers; shared by the translation units that
// implement entry points taking a handle.
#pragma once
#include <vector>

#include "host.h"

struct tgbm_model {
    std::vector<tgbm::Tree> trees;
};
