// tt/random.h — TEST-SIDE STAND-IN (see tt/exception.h in this directory): the generator of tensor/random.cpp:26-63,
// state = splitmix64(seed), outputs = xorshift64 with shifts 13, 7, 17.
#ifndef TT_STANDIN_RANDOM_H_
#define TT_STANDIN_RANDOM_H_

#include <cstdint>

namespace tinytensor {

class Generator {
public:
    Generator(uint64_t seed) {    // NOLINT(*-explicit-*): the reference's constructor converts too
        uint64_t z = seed + 0x9E3779B97F4A7C15ULL;
        z = (z ^ (z >> 30U)) * 0xBF58476D1CE4E5B9ULL;
        z = (z ^ (z >> 27U)) * 0x94D049BB133111EBULL;
        state = z ^ (z >> 31U);
    }
    static auto from_state(uint64_t s) -> Generator {
        Generator g(0);
        g.state = s;
        return g;
    }
    auto operator()() noexcept -> uint64_t {
        state ^= state << 13U;
        state ^= state >> 7U;
        state ^= state << 17U;
        return state;
    }
    void set_state(uint64_t s) { state = s; }

private:
    uint64_t state;
};

}    // namespace tinytensor

#endif    // TT_STANDIN_RANDOM_H_
