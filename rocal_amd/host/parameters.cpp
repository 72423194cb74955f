#include "parameters.h"

ParameterFactory *ParameterFactory::_instance = nullptr;
std::mutex ParameterFactory::_instance_mutex;

ParameterFactory::ParameterFactory() { generate_seed(); }

ParameterFactory *ParameterFactory::instance() {
    std::lock_guard<std::mutex> g(_instance_mutex);
    if (!_instance) _instance = new ParameterFactory();
    return _instance;
}

ParameterFactory::~ParameterFactory() {
    for (auto &p : _registry) std::visit([](auto *q) { delete q; }, p);
}

void ParameterFactory::renew_parameters() {
    for (auto &p : _registry) std::visit([](auto *q) { q->renew(); }, p);
}

void ParameterFactory::generate_seed() {
    std::random_device rd;
    set_seed(rd());
}

// parameter_factory.cpp:112-117: MAX_SEEDS 64-bit slots filled by std::seed_seq{seed}.generate (each slot
// receives one 32-bit output).
void ParameterFactory::set_seed(unsigned seed) {
    _seed = seed;
    _seed_vector.assign(MAX_SEEDS, 0);
    std::seed_seq seq{seed};
    seq.generate(_seed_vector.begin(), _seed_vector.end());  // the read position is kept, as in the reference
}

int64_t ParameterFactory::get_seed_from_seedsequence() {
    const int64_t s = _seed_vector[_seed_idx];
    _seed_idx = (_seed_idx + 1) % MAX_SEEDS;
    return s;
}

IntParam *ParameterFactory::create_uniform_int_rand_param(int start, int end) {
    auto *p = new UniformRand<int>(start, end, (unsigned)get_seed_from_seedsequence());
    _registry.insert(p);
    return new IntParam(p, RocalParameterType::RANDOM_UNIFORM);
}

FloatParam *ParameterFactory::create_uniform_float_rand_param(float start, float end) {
    auto *p = new UniformRand<float>(start, end, (unsigned)get_seed_from_seedsequence());
    _registry.insert(p);
    return new FloatParam(p, RocalParameterType::RANDOM_UNIFORM);
}

IntParam *ParameterFactory::create_custom_int_rand_param(const int *values, const double *frequencies, size_t size) {
    auto *p = new CustomRand<int>(values, frequencies, size, (unsigned)get_seed_from_seedsequence());
    _registry.insert(p);
    return new IntParam(p, RocalParameterType::RANDOM_CUSTOM);
}

FloatParam *ParameterFactory::create_custom_float_rand_param(const float *values, const double *frequencies, size_t size) {
    auto *p = new CustomRand<float>(values, frequencies, size, (unsigned)get_seed_from_seedsequence());
    _registry.insert(p);
    return new FloatParam(p, RocalParameterType::RANDOM_CUSTOM);
}

IntParam *ParameterFactory::create_single_value_int_param(int value) {
    auto *p = new SimpleParameter<int>(value);
    _registry.insert(p);
    return new IntParam(p, RocalParameterType::DETERMINISTIC);
}

FloatParam *ParameterFactory::create_single_value_float_param(float value) {
    auto *p = new SimpleParameter<float>(value);
    _registry.insert(p);
    return new FloatParam(p, RocalParameterType::DETERMINISTIC);
}
