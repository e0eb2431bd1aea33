// packed_func.h -- type-erased functions and the global function registry.
//
// Interface of the reference's include/base/packedfunc.h:22-240 (TypeCode, Args, PackedFunc, RetValue) and
// include/base/registry.h:13-61 (Registry::Global().Set / Get, KXC_REGISTER_GLOBAL(name).set_body(f)): the face the
// reference's language bindings call through.  Registered here (host/src/packed_func.cc), with the argument order of
// src/base/device_api.cc:442-658: the device_api.* functions for both back ends, target.Build,
// device.DetectAndRegister (device_info.hip.<i>.name / .memory / .compute_capability), and
// kxc.relay.transform.lower_to_exec_plan_json[_file] (src/relay/transforms/multi_device.cc:524-539) with their
// single-device runners kxc.hip.execute_plan_json[_file].
//
// Values are owned by the Args object (the reference passes borrowed unions; owning them removes the lifetime rules
// without changing what a callee sees): an integer, a double, text, an object handle, a raw pointer or nothing.
#pragma once

#include <functional>

#include "kxc/device_api.h"

namespace kxc {

enum TypeCode : int { kInt = 0, kFloat = 1, kString = 2, kObjectRef = 3, kNull = 4, kHandle = 5 };

struct Value {
    int64_t v_int = 0;
    double v_float = 0.0;
    std::string v_str;
    ObjectRef v_object;
    void* v_handle = nullptr;
};

// A Device travels as an object argument (the reference's Device is an object handle, include/base/device.h:20-62).
struct DeviceObj : Object {
    Device device;
};

class Args {
public:
    Args() = default;
    int size() const { return static_cast<int>(values_.size()); }
    const Value& operator[](int index) const { return values_.at(Checked(index)); }
    TypeCode type_code(int index) const { return codes_.at(Checked(index)); }

    void Push(int64_t v) { Value x; x.v_int = v; Add(x, kInt); }
    void Push(int v) { Push(static_cast<int64_t>(v)); }
    void Push(bool v) { Push(static_cast<int64_t>(v)); }
    void Push(double v) { Value x; x.v_float = v; Add(x, kFloat); }
    void Push(const std::string& v) { Value x; x.v_str = v; Add(x, kString); }
    void Push(const char* v) { Push(std::string(v ? v : "")); }
    void Push(const ObjectRef& v) { Value x; x.v_object = v; Add(x, v.defined() ? kObjectRef : kNull); }
    void Push(void* v) { Value x; x.v_handle = v; Add(x, kHandle); }
    void Push(const Device& d) {
        auto node = std::make_shared<DeviceObj>();
        node->device = d;
        Push(ObjectRef(Ref<DeviceObj>(node)));
    }
    template <typename U, typename = typename std::enable_if<std::is_base_of<Object, U>::value>::type>
    void Push(const Ref<U>& v) { Push(ObjectRef(v)); }

private:
    int Checked(int index) const {
        if (index < 0 || index >= size()) throw std::out_of_range("index out of range");
        return index;
    }
    void Add(const Value& v, TypeCode c) { values_.push_back(v); codes_.push_back(c); }
    std::vector<Value> values_;
    std::vector<TypeCode> codes_;
};

// Typed reads of one argument; the messages are the reference's (include/base/packedfunc.h:261-300).
template <typename T, typename Enable = void>
struct ArgConverter;
template <> struct ArgConverter<int64_t> {
    static int64_t From(const Value& v, TypeCode t) {
        if (t != kInt) throw std::runtime_error("Type mismatch, expected int64_t");
        return v.v_int;
    }
};
template <> struct ArgConverter<int> {
    static int From(const Value& v, TypeCode t) {
        if (t != kInt) throw std::runtime_error("Type mismatch, expected int");
        return static_cast<int>(v.v_int);
    }
};
template <> struct ArgConverter<bool> {
    static bool From(const Value& v, TypeCode t) {
        if (t != kInt) throw std::runtime_error("Type mismatch, expected bool (int)");
        return v.v_int != 0;
    }
};
template <> struct ArgConverter<double> {
    static double From(const Value& v, TypeCode t) {
        if (t != kFloat) throw std::runtime_error("Type mismatch, expected double");
        return v.v_float;
    }
};
template <> struct ArgConverter<std::string> {
    static std::string From(const Value& v, TypeCode t) {
        if (t != kString) throw std::runtime_error("Type mismatch, expected string");
        return v.v_str;
    }
};
template <> struct ArgConverter<ObjectRef> {
    static ObjectRef From(const Value& v, TypeCode t) {
        if (t != kObjectRef) throw std::runtime_error("Type mismatch, expected ObjectRef");
        return v.v_object;
    }
};
template <> struct ArgConverter<void*> {
    static void* From(const Value& v, TypeCode t) {
        if (t != kHandle) throw std::runtime_error("Type mismatch, expected Handle");
        return v.v_handle;
    }
};
template <> struct ArgConverter<Device> {
    static Device From(const Value& v, TypeCode t) {
        const DeviceObj* d = t == kObjectRef ? v.v_object.As<DeviceObj>() : nullptr;
        if (!d) throw std::runtime_error("Type mismatch, expected ObjectRef");
        return d->device;
    }
};

class PackedFunc {
public:
    using Body = std::function<void(Args, RetValue*)>;
    PackedFunc() = default;
    explicit PackedFunc(Body body) : body_(std::make_shared<Body>(std::move(body))) {}
    bool defined() const { return static_cast<bool>(body_); }
    void operator()(Args args, RetValue* rv) const {
        if (!body_) throw std::runtime_error("PackedFunc is empty");
        (*body_)(std::move(args), rv);
    }
    template <typename... T>
    RetValue operator()(T&&... values) const {
        Args args;
        (args.Push(std::forward<T>(values)), ...);
        RetValue rv;
        (*this)(std::move(args), &rv);
        return rv;
    }

private:
    std::shared_ptr<Body> body_;
};

class Registry {
public:
    static Registry& Global();
    // Registering a name twice throws "Function <name> is already registered."
    void Set(const std::string& name, PackedFunc func);
    // An absent name gives an empty PackedFunc (defined() == false).
    PackedFunc Get(const std::string& name) const;
    std::vector<std::string> ListNames() const;

private:
    Registry() = default;
    std::map<std::string, PackedFunc> functions_;
};

class RegistryEntry {
public:
    explicit RegistryEntry(std::string name) : name_(std::move(name)) {}
    RegistryEntry& set_body(PackedFunc f) {
        Registry::Global().Set(name_, std::move(f));
        return *this;
    }

private:
    std::string name_;
};

#define KXC_STR_CONCAT_(x, y) x##y
#define KXC_STR_CONCAT(x, y) KXC_STR_CONCAT_(x, y)
#define KXC_REGISTER_GLOBAL(Name) \
    static ::kxc::RegistryEntry KXC_STR_CONCAT(kxc_reg_entry_, __COUNTER__) = ::kxc::RegistryEntry(Name)

// Registers device_info.hip.<i>.{name,memory,compute_capability} for every visible GPU (once); the counterpart of
// DetectAndRegisterDevices (src/base/device_api.cc:388-438).
void DetectAndRegisterDevices();

}  // namespace kxc
