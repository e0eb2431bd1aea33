// base.h -- handle type, containers and small utilities of the host layer.
//
// The host layer mirrors the operator / compile / run interface of the kxc compiler
// (names, argument meaning and error behaviour), re-implemented for the HIP backend: graph
// building (relay.h, op.h), TE compute definitions (te.h, topi.h), lowering to TIR (lower.h),
// code generators (codegen_c.h for the host, codegen_hip.h for gfx950), device API, compile
// configuration and the CompiledModule whose Run(void* packed_args[]) enqueues a launch plan.
#pragma once

#include <cstdint>
#include <initializer_list>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

namespace kxc {

// Common base of every node a handle points to, so that code written against the reference can key maps by
// `const Object*` and pass any handle where an ObjectRef is expected (include/base/object.h:68-183).
struct Object {
    virtual ~Object() = default;
};

// Shared, nullable handle to an immutable-by-convention node.  `defined()`, `get()`, `As<T>()` and
// `operator->` follow the reference's ObjectRef vocabulary (include/base/object.h:115-183).
template <typename NodeT>
class Ref {
public:
    Ref() = default;
    explicit Ref(std::shared_ptr<NodeT> p) : ptr_(std::move(p)) {}
    bool defined() const { return static_cast<bool>(ptr_); }
    NodeT* get() const { return ptr_.get(); }
    NodeT* operator->() const { return ptr_.get(); }
    template <typename T>
    const T* As() const { return dynamic_cast<const T*>(ptr_.get()); }
    bool same_as(const Ref& o) const { return ptr_ == o.ptr_; }
    const std::shared_ptr<NodeT>& shared() const { return ptr_; }

protected:
    std::shared_ptr<NodeT> ptr_;
};

// Handle to any node: every Ref<T> with T derived from Object converts to it.
class ObjectRef : public Ref<Object> {
public:
    ObjectRef() = default;
    template <typename U, typename = typename std::enable_if<std::is_base_of<Object, U>::value>::type>
    ObjectRef(const Ref<U>& other) : Ref<Object>(std::shared_ptr<Object>(other.shared())) {}
};

// Array<T>: a value-semantics vector with the reference's push_back/size/[] surface
// (include/base/container.h).
template <typename T>
class Array : public std::vector<T> {
public:
    using std::vector<T>::vector;
    Array() = default;
    Array(std::initializer_list<T> init) : std::vector<T>(init) {}
    Array(const std::vector<T>& v) : std::vector<T>(v) {}
};

using String = std::string;

template <typename K, typename V>
class Map : public std::map<K, V> {
public:
    void Set(const K& k, const V& v) { (*this)[k] = v; }
};

inline int64_t Product(const std::vector<int64_t>& v) {
    int64_t p = 1;
    for (auto d : v) p *= d;
    return p;
}

}  // namespace kxc
