// Host-side parameter system of the augmentation hot path, with rocAL's class names and laws.
//
// What must match the reference bit for bit is the LAW of each generator (one std::mt19937 per
// parameter, one draw per value, the double-precision map to [start,end], truncation for ints),
// because the per-sample values it produces are inputs of the kernels:
//   UniformRand  rocAL/include/parameters/parameter_random.h:37-118
//   CustomRand   rocAL/include/parameters/parameter_random.h:120-238
//   SimpleParameter rocAL/include/parameters/parameter_simple.h:26-71
//   ParameterFactory rocAL/include/parameters/parameter_factory.h:73-118, source/parameters/parameter_factory.cpp:64-160
//   ParameterVX  rocAL/include/parameters/parameter_vx.h:32-122  (the vx_array becomes a host vector here;
//                its contents reach the device through the per-batch parameter table of the C ABI)
#pragma once
#include <algorithm>
#include <cstdint>
#include <mutex>
#include <numeric>
#include <random>
#include <set>
#include <variant>
#include <vector>

#include "exception.h"

template <typename T>
class Parameter {
   public:
    virtual ~Parameter() {}
    virtual T default_value() const = 0;
    virtual T get() = 0;
    virtual void renew() {}
    virtual void create_array(unsigned) {}
    virtual std::vector<T> get_array() { return {}; }
    virtual bool single_value() const = 0;
};

template <typename T>
class SimpleParameter : public Parameter<T> {
   public:
    explicit SimpleParameter(T value) : _val(value) {}
    T default_value() const override { return _val; }
    T get() override { return _val; }
    std::vector<T> get_array() override { return _values; }
    // As the reference: once the array exists, update() re-fills it with the value held before the call
    // and does not change that value (parameter_simple.h:45-56).
    int update(T new_val) {
        if (_values.empty())
            _val = new_val;
        else
            std::fill(_values.begin(), _values.end(), _val);
        return 0;
    }
    void create_array(unsigned n) override {
        if (_values.empty()) _values.resize(n);
        update(_val);
    }
    bool single_value() const override { return true; }

   private:
    T _val;
    std::vector<T> _values;
};

template <typename T>
class UniformRand : public Parameter<T> {
   public:
    UniformRand(T start, T end, unsigned seed = 0) : _engine(seed) {
        update(start, end);
        renew();
    }
    explicit UniformRand(T start, unsigned seed = 0) : UniformRand(start, start, seed) {}
    T default_value() const override { return static_cast<T>((_lo + _hi) / static_cast<T>(2)); }
    T get() override { return _current; }
    std::vector<T> get_array() override { return _values; }
    bool single_value() const override { return _lo == _hi; }
    int update(T start, T end) {
        std::lock_guard<std::mutex> g(_mutex);
        _lo = start;
        _hi = end < start ? start : end;
        return 0;
    }
    // One engine draw per value even when the range is a single point (the draw happens first).
    void renew_value() {
        std::lock_guard<std::mutex> g(_mutex);
        renew_value_unlocked();
    }
    // For a caller that draws a whole batch from this parameter (the crop-window laws): it takes mutex() once for the batch
    // and then draws with renew_value_unlocked(), which is renew() + get() of a parameter without an array.
    std::mutex &mutex() { return _mutex; }
    bool has_array() const { return !_values.empty(); }
    T renew_value_unlocked() {
        const auto raw = _engine();
        if (single_value())
            _current = _lo;
        else
            _current = static_cast<T>(((double)raw / (double)_engine.max()) * ((double)_hi - (double)_lo) + (double)_lo);
        return _current;
    }
    void renew() override {
        if (_values.empty()) {
            renew_value();
            return;
        }
        for (auto &v : _values) {
            renew_value();
            v = _current;
        }
    }
    void create_array(unsigned n) override {
        if (_values.empty()) _values.resize(n);
    }

   private:
    T _lo{}, _hi{}, _current{};
    std::vector<T> _values;
    std::mt19937 _engine;
    std::mutex _mutex;
};

template <typename T>
class CustomRand : public Parameter<T> {
   public:
    CustomRand(const T values[], const double frequencies[], size_t size, unsigned seed = 0) : _engine(seed) {
        update(values, frequencies, size);
        renew();
    }
    int update(const T values[], const double frequencies[], size_t size) {
        std::lock_guard<std::mutex> g(_mutex);
        if (size == 0) return -1;
        _choices.assign(values, values + size);
        // Frequencies that are negative or zero are dropped by compaction, exactly as the reference's
        // std::copy_if does (its predicate returns the frequency itself, read as a bool): the kept entries
        // move to the front and the tail keeps its old contents.
        _prob.assign(frequencies, frequencies + size);
        double sum = 0;
        size_t w = 0;
        for (size_t r = 0; r < size; r++)
            if (_prob[r] > 0) {
                sum += _prob[r];
                _prob[w++] = _prob[r];
            }
        for (auto &p : _prob) p = p / sum;
        // std::inner_product with an int initial value accumulates in int (parameter_random.h:160-163).
        int acc = 0;
        for (size_t i = 0; i < size; i++) acc = acc + _choices[i] * _prob[i];
        _mean = acc;
        _cdf.assign(size, 0.0);
        std::partial_sum(_prob.begin(), _prob.end(), _cdf.begin());
        return 0;
    }
    T default_value() const override { return static_cast<T>(_mean); }
    T get() override { return _current; }
    std::vector<T> get_array() override { return _values; }
    bool single_value() const override { return _choices.size() == 1; }
    void renew_value() {
        std::lock_guard<std::mutex> g(_mutex);
        if (single_value()) {
            _current = _choices[0];
            return;
        }
        const double u = (double)_engine() / (double)_engine.max();
        const size_t idx = std::upper_bound(_cdf.begin(), _cdf.end(), u) - _cdf.begin();
        _current = _choices[idx];
    }
    void renew() override {
        if (_values.empty()) {
            renew_value();
            return;
        }
        for (auto &v : _values) {
            renew_value();
            v = _current;
        }
    }
    void create_array(unsigned n) override {
        if (_values.empty()) _values.resize(n);
    }

   private:
    std::vector<T> _choices;
    std::vector<double> _prob, _cdf;
    double _mean = 0;
    T _current{};
    std::vector<T> _values;
    std::mt19937 _engine;
    std::mutex _mutex;
};

enum class RocalParameterType { DETERMINISTIC = 0, RANDOM_UNIFORM, RANDOM_CUSTOM };

struct IntParam {
    IntParam(Parameter<int> *c, RocalParameterType t) : core(c), type(t) {}
    Parameter<int> *core;
    const RocalParameterType type;
};
struct FloatParam {
    FloatParam(Parameter<float> *c, RocalParameterType t) : core(c), type(t) {}
    Parameter<float> *core;
    const RocalParameterType type;
};
inline Parameter<int> *core(IntParam *p) { return p ? p->core : nullptr; }
inline Parameter<float> *core(FloatParam *p) { return p ? p->core : nullptr; }

// Process-wide registry of parameters. renew_parameters() is called once per batch by the pipeline
// (rocAL/source/pipeline/master_graph.cpp:408) and renews EVERY registered parameter once.
class ParameterFactory {
   public:
    static constexpr int MAX_SEEDS = 1024;
    static ParameterFactory *instance();
    ~ParameterFactory();
    void renew_parameters();
    void set_seed(unsigned seed);  // also derives MAX_SEEDS values with std::seed_seq{seed}
    unsigned get_seed() { return (unsigned)_seed; }
    void generate_seed();
    int64_t get_seed_from_seedsequence();

    // Default parameters of nodes use the factory seed itself, user-created ones the seed sequence.
    template <typename T>
    Parameter<T> *create_uniform_rand_param(T start, T end) {
        auto *p = new UniformRand<T>(start, end, (unsigned)_seed);
        _registry.insert(p);
        return p;
    }
    template <typename T>
    Parameter<T> *create_single_value_param(T value) {
        auto *p = new SimpleParameter<T>(value);
        _registry.insert(p);
        return p;
    }
    template <typename T>
    void destroy_param(Parameter<T> *p) {
        _registry.erase(p);
        delete p;
    }
    IntParam *create_uniform_int_rand_param(int start, int end);
    FloatParam *create_uniform_float_rand_param(float start, float end);
    IntParam *create_custom_int_rand_param(const int *values, const double *frequencies, size_t size);
    FloatParam *create_custom_float_rand_param(const float *values, const double *frequencies, size_t size);
    IntParam *create_single_value_int_param(int value);
    FloatParam *create_single_value_float_param(float value);

   private:
    ParameterFactory();
    using Any = std::variant<Parameter<int> *, Parameter<float> *>;
    long long unsigned _seed = 0;
    std::set<Any> _registry;
    std::vector<int64_t> _seed_vector;
    size_t _seed_idx = 0;
    static ParameterFactory *_instance;
    static std::mutex _instance_mutex;
};

// Batch-sized view of one parameter: what the reference keeps in a vx_array of N items and refreshes
// in update_node(). values() is what is handed to rmx_update_*().
template <typename T>
class ParameterVX {
   public:
    ParameterVX(T default_range_start, T default_range_end)
        : _param(ParameterFactory::instance()->create_uniform_rand_param<T>(default_range_start, default_range_end)) {}
    void create_array(unsigned batch_size) {
        _batch_size = batch_size;
        _param->create_array(batch_size);
        update_array();
    }
    void set_param(Parameter<T> *p) {
        if (!p) return;  // keep the default random parameter
        ParameterFactory::instance()->destroy_param(_param);
        _param = p;
    }
    void set_param(T value) {
        ParameterFactory::instance()->destroy_param(_param);
        _param = ParameterFactory::instance()->create_single_value_param(value);
    }
    T default_value() { return _param->default_value(); }
    void update_array() {
        _values = _param->get_array();
        if (_values.size() != _batch_size) THROW("ParameterVX: parameter array has " + TOSTR(_values.size()) + " items for a batch of " + TOSTR(_batch_size));
    }
    T renew() {
        _param->renew();
        return _param->get();
    }
    std::vector<T> get_array() { return _param->get_array(); }
    const std::vector<T> &values() const { return _values; }

   private:
    Parameter<T> *_param;
    std::vector<T> _values;
    unsigned _batch_size = 0;
};
