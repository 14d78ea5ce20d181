// Host-side mirror of the reference's common module: error values, MaybeDyn
// sentinels, TensorLayout accessors and the small validators every Args::meta
// uses (operators/src/common/{error,maybe_dyn,tensor,mod}.rs).
#pragma once
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <list>
#include <mutex>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../kernels/params.h"
#include "ophip.h"

namespace ophip {

// SchemeError / LaunchError (common/error.rs:14-39): a kind plus free text.
struct Error {
    int kind;
    std::string info;
};

inline Error type_not_support(std::string s) { return {OPHIP_TYPE_NOT_SUPPORT, std::move(s)}; }
inline Error type_mismatch(std::string s) { return {OPHIP_TYPE_MISMATCH, std::move(s)}; }
inline Error rank_not_support(std::string s) { return {OPHIP_RANK_NOT_SUPPORT, std::move(s)}; }
inline Error rank_mismatch(std::string s) { return {OPHIP_RANK_MISMATCH, std::move(s)}; }
inline Error shape_not_support(std::string s) { return {OPHIP_SHAPE_NOT_SUPPORT, std::move(s)}; }
inline Error shape_mismatch(std::string s) { return {OPHIP_SHAPE_MISMATCH, std::move(s)}; }
inline Error strides_not_support(std::string s) { return {OPHIP_STRIDES_NOT_SUPPORT, std::move(s)}; }
inline Error args_not_support(std::string s) { return {OPHIP_ARGS_NOT_SUPPORT, std::move(s)}; }
inline Error dyn_not_support(std::string s) { return {OPHIP_DYNAMIC_NOT_SUPPORT, std::move(s)}; }
inline Error execution_failed(std::string s) { return {OPHIP_EXECUTION_FAILED, std::move(s)}; }

void set_last_error(const std::string &s);

// Runs f, turning any Error (or stray C++ exception) into a status code: nothing
// unwinds across the C ABI.
template <class F>
int guard(F &&f) noexcept {
    try {
        f();
        set_last_error("");
        return OPHIP_OK;
    } catch (const Error &e) {
        set_last_error(std::string(ophip_status_name(e.kind)) + (e.info.empty() ? "" : ": " + e.info));
        return e.kind;
    } catch (const std::exception &e) {
        set_last_error(std::string("ExecutionFailed: ") + e.what());
        return OPHIP_EXECUTION_FAILED;
    } catch (...) {
        set_last_error("ExecutionFailed: unknown exception");
        return OPHIP_EXECUTION_FAILED;
    }
}

// MaybeDyn (common/maybe_dyn.rs:6-37)
inline bool is_dyn(size_t v) { return v == OPHIP_DYN_USIZE; }
inline bool is_dyn(ptrdiff_t v) { return v == OPHIP_DYN_ISIZE; }
inline bool is_dyn(float v) { return std::isinf(v) && v > 0; }

// get_static! (common/maybe_dyn.rs:105-114)
template <class T>
inline T static_of(T v) {
    if (is_dyn(v)) throw dyn_not_support("");
    return v;
}

// utils::dim_distinct (common/mod.rs:57-61) on MaybeDyn::merge (maybe_dyn.rs:76-91)
inline size_t dim_distinct(std::initializer_list<size_t> dims) {
    auto it = dims.begin();
    size_t acc = *it++;
    for (; it != dims.end(); ++it) {
        if (is_dyn(*it)) continue;
        if (is_dyn(acc)) acc = *it;
        else if (acc != *it) throw shape_mismatch("dims are not distinct");
    }
    return acc;
}

// utils::type_distinct (common/mod.rs:38-49)
inline uint64_t type_distinct(std::initializer_list<uint64_t> dts) {
    const uint64_t dt = *dts.begin();
    for (uint64_t d : dts)
        if (d != dt) throw type_mismatch("data types are not distinct");
    return dt;
}

// utils::rank_error (common/mod.rs:51-54)
inline Error rank_error(const char *arg, size_t expected, size_t actual) {
    return rank_not_support(std::string(arg) + ".ndim = " + std::to_string(actual) + ", " +
                            std::to_string(expected) + " expected");
}

// A layout of non-zero rank has to bring its shape and strides (a binding that leaves the pointers null gets a status).
inline void expect_arrays(const ophip_tensor_layout &l) {
    if (l.ndim != 0 && (!l.shape || !l.strides)) throw args_not_support("a layout without shape or strides");
}
inline void expect_rank(const ophip_tensor_layout &l, const char *name, size_t rank) {
    if (l.ndim != rank) throw rank_error(name, rank, l.ndim);
    expect_arrays(l);
}

inline bool is_float_dtype(uint64_t dt) {
    return dt == OPHIP_DT_F16 || dt == OPHIP_DT_BF16 || dt == OPHIP_DT_F32 || dt == OPHIP_DT_F64;
}
inline bool is_unsigned_dtype(uint64_t dt) {
    return dt == OPHIP_DT_U8 || dt == OPHIP_DT_U16 || dt == OPHIP_DT_U32 || dt == OPHIP_DT_U64;
}

// Division of any 32-bit n by a launch-time constant d >= 1 (the kernels' `fastdiv`):
// q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(m, n).
inline FastDivU32 make_fastdiv(uint32_t d) {
    FastDivU32 f{};
    f.d = d;
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    f.m = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l == 0 ? 0 : l - 1;
    return f;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool mult16(ptrdiff_t v) { return (v & 15) == 0; }

// f32 -> f16 -> f32 (round to nearest even), for the scalars the reference rounds to f16
float round_to_f16(float f);
float round_to_bf16(float f);  // nearest even; NaN and infinity unchanged

// Least-recently-used map guarded by a mutex: the shape of the reference's
// Mutex<LruCache<SchemeKey, Scheme>> (e.g. rms_norm/cuda/mod.rs:14-17).
template <class K, class V, class Hash = std::hash<K>>
class LruCache {
   public:
    explicit LruCache(size_t cap) : cap_(cap ? cap : 1) {}
    template <class Make>
    V get_or_insert(const K &key, Make &&make) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = map_.find(key);
        if (it != map_.end()) {
            order_.splice(order_.begin(), order_, it->second);
            return it->second->second;
        }
        V v = make();
        order_.emplace_front(key, v);
        map_[key] = order_.begin();
        if (map_.size() > cap_) {
            map_.erase(order_.back().first);
            order_.pop_back();
        }
        return v;
    }
    size_t size() {
        std::lock_guard<std::mutex> lock(mu_);
        return map_.size();
    }

   private:
    size_t cap_;
    std::mutex mu_;
    std::list<std::pair<K, V>> order_;
    std::unordered_map<K, typename std::list<std::pair<K, V>>::iterator, Hash> map_;
};

}  // namespace ophip
