// Stand-in for the part of OpenVINO's developer API that the "HIP" plugin sources use.
//
// The plugin (plugin/src/*.cpp) is written against OpenVINO's own headers -- "openvino/runtime/
// iplugin.hpp", "openvino/core/node.hpp", ... -- and names only declarations of namespace ov.  Where
// the OpenVINO developer package is installed, CMake points the include path at it and this
// directory is not used at all.  Where it is not (this repository's own build and tests), the
// include path points here: every header under standin/openvino/ forwards to this file, which
// declares the same classes with the same member signatures, as far as the plugin touches them
// (the list is the one the reference plugin uses, modules/nvidia_plugin/src/cuda_plugin.hpp:25-55,
// cuda_compiled_model.hpp:42-57, cuda_infer_request.hpp:42-55, cuda_async_infer_request.cpp:26-61,
// cuda_variable_state.hpp:31-105), and gives them a small working implementation: a graph of
// nodes, host tensors, an infer-request base with its tensor bookkeeping, the staged asynchronous
// pipeline with cancel and stop_and_wait, a text serialisation.  It plays the part ov::Core plays
// for the real plugin; it is not OpenVINO and proves structure, not binary compatibility.
#pragma once

#include <algorithm>
#include <any>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <exception>
#include <functional>
#include <future>
#include <istream>
#include <map>
#include <memory>
#include <mutex>
#include <ostream>
#include <set>
#include <sstream>
#include <stdexcept>
#include <string>
#include <thread>
#include <typeinfo>
#include <unordered_set>
#include <utility>
#include <vector>

#define OPENVINO_STANDIN 1
#define OPENVINO_PLUGIN_API __attribute__((visibility("default")))

namespace ov {

// ------------------------------------------------------------------------------ errors
class Exception : public std::runtime_error {
public:
    explicit Exception(const std::string& what) : std::runtime_error(what) {}
};
class NotImplemented : public Exception {
public:
    explicit NotImplemented(const std::string& what) : Exception(what) {}
};
class Cancelled : public Exception {
public:
    explicit Cancelled(const std::string& what) : Exception(what) {}
};
class Busy : public Exception {
public:
    explicit Busy(const std::string& what) : Exception(what) {}
};

namespace standin {
template <typename... Args>
std::string concat(Args&&... args) {
    std::ostringstream ss;
    (void)std::initializer_list<int>{((ss << args), 0)...};
    return ss.str();
}
}  // namespace standin

#define OPENVINO_THROW(...) \
    throw ::ov::Exception(::ov::standin::concat("Exception from ", __FILE__, ":", __LINE__, ":\n", __VA_ARGS__))
#define OPENVINO_ASSERT(cond, ...)                                                                              \
    do {                                                                                                        \
        if (!(cond))                                                                                            \
            throw ::ov::Exception(::ov::standin::concat("Check '", #cond, "' failed at ", __FILE__, ":", __LINE__, \
                                                        ":\n", ##__VA_ARGS__));                                  \
    } while (0)
#define OPENVINO_NOT_IMPLEMENTED \
    throw ::ov::NotImplemented(::ov::standin::concat("Not Implemented at ", __FILE__, ":", __LINE__))
#define OPENVINO_THROW_NOT_IMPLEMENTED(...) \
    throw ::ov::NotImplemented(::ov::standin::concat("Not Implemented at ", __FILE__, ":", __LINE__, ":\n", __VA_ARGS__))

// ------------------------------------------------------------------------------ Any
// Holds any copyable value; as<T>() also reads numbers and booleans out of strings, as properties
// arrive from configuration files.
class Any {
public:
    Any() = default;
    template <typename T, typename = std::enable_if_t<!std::is_same_v<std::decay_t<T>, Any>>>
    Any(T&& value) : value_(normalise(std::forward<T>(value))) {}
    bool empty() const { return !value_.has_value(); }
    template <typename T>
    bool is() const {
        return value_.type() == typeid(T);
    }
    template <typename T>
    T as() const {
        if (auto p = std::any_cast<T>(&value_)) return *p;
        if constexpr (std::is_same_v<T, std::string>) {
            if (auto p = std::any_cast<bool>(&value_)) return *p ? "YES" : "NO";
            if (auto p = std::any_cast<int64_t>(&value_)) return std::to_string(*p);
            if (auto p = std::any_cast<double>(&value_)) return std::to_string(*p);
        } else if constexpr (std::is_same_v<T, bool>) {
            if (auto p = std::any_cast<std::string>(&value_)) {
                if (*p == "YES" || *p == "true" || *p == "1") return true;
                if (*p == "NO" || *p == "false" || *p == "0") return false;
            }
            if (auto p = std::any_cast<int64_t>(&value_)) return *p != 0;
        } else if constexpr (std::is_arithmetic_v<T>) {
            if (auto p = std::any_cast<int64_t>(&value_)) return static_cast<T>(*p);
            if (auto p = std::any_cast<double>(&value_)) return static_cast<T>(*p);
            if (auto p = std::any_cast<bool>(&value_)) return static_cast<T>(*p);
            if (auto p = std::any_cast<std::string>(&value_)) {
                size_t pos = 0;
                try {
                    if constexpr (std::is_floating_point_v<T>) {
                        const double x = std::stod(*p, &pos);
                        if (pos == p->size()) return static_cast<T>(x);
                    } else {
                        const long long x = std::stoll(*p, &pos);
                        if (pos == p->size()) return static_cast<T>(x);
                    }
                } catch (const std::exception&) {
                }
            }
        }
        throw Exception(std::string("Bad cast from: ") + value_.type().name() + " to: " + typeid(T).name());
    }

private:
    template <typename T>
    static std::any normalise(T&& v) {
        using D = std::decay_t<T>;
        if constexpr (std::is_same_v<D, const char*> || std::is_same_v<D, char*>)
            return std::string(v);
        else if constexpr (std::is_same_v<D, bool>)
            return v;
        else if constexpr (std::is_integral_v<D>)
            return static_cast<int64_t>(v);
        else if constexpr (std::is_floating_point_v<D>)
            return static_cast<double>(v);
        else
            return D(std::forward<T>(v));
    }
    std::any value_;
};
using AnyMap = std::map<std::string, Any>;

// ------------------------------------------------------------------------------ element types
namespace element {
enum class Type_t { dynamic, boolean, bf16, f16, f32, f64, i8, i16, i32, i64, u8, u16, u32, u64 };
class Type {
public:
    constexpr Type() = default;
    constexpr Type(Type_t t) : t_(t) {}
    constexpr operator Type_t() const { return t_; }
    size_t size() const { return (bitwidth() + 7) / 8; }
    size_t bitwidth() const {
        switch (t_) {
            case Type_t::boolean:
            case Type_t::i8:
            case Type_t::u8: return 8;
            case Type_t::bf16:
            case Type_t::f16:
            case Type_t::i16:
            case Type_t::u16: return 16;
            case Type_t::f32:
            case Type_t::i32:
            case Type_t::u32: return 32;
            case Type_t::f64:
            case Type_t::i64:
            case Type_t::u64: return 64;
            default: return 0;
        }
    }
    bool is_real() const { return t_ == Type_t::bf16 || t_ == Type_t::f16 || t_ == Type_t::f32 || t_ == Type_t::f64; }
    bool is_dynamic() const { return t_ == Type_t::dynamic; }
    bool is_static() const { return !is_dynamic(); }
    bool compatible(const Type& other) const { return is_dynamic() || other.is_dynamic() || t_ == other.t_; }
    std::string get_type_name() const {
        static const char* names[] = {"dynamic", "boolean", "bf16", "f16", "f32", "f64", "i8",
                                      "i16",     "i32",     "i64",  "u8",  "u16", "u32", "u64"};
        return names[static_cast<int>(t_)];
    }
    std::string to_string() const { return get_type_name(); }
    friend bool operator==(const Type& a, const Type& b) { return a.t_ == b.t_; }
    friend bool operator!=(const Type& a, const Type& b) { return a.t_ != b.t_; }
    friend bool operator<(const Type& a, const Type& b) { return a.t_ < b.t_; }

private:
    Type_t t_ = Type_t::dynamic;
};
inline std::ostream& operator<<(std::ostream& os, const Type& t) { return os << t.get_type_name(); }
constexpr Type dynamic(Type_t::dynamic);
constexpr Type boolean(Type_t::boolean);
constexpr Type bf16(Type_t::bf16);
constexpr Type f16(Type_t::f16);
constexpr Type f32(Type_t::f32);
constexpr Type f64(Type_t::f64);
constexpr Type i8(Type_t::i8);
constexpr Type i32(Type_t::i32);
constexpr Type i64(Type_t::i64);
constexpr Type u8(Type_t::u8);
constexpr Type u32(Type_t::u32);
constexpr Type u64(Type_t::u64);
inline Type type_from_name(const std::string& name) {
    for (Type_t t : {Type_t::dynamic, Type_t::boolean, Type_t::bf16, Type_t::f16, Type_t::f32, Type_t::f64, Type_t::i8,
                     Type_t::i16, Type_t::i32, Type_t::i64, Type_t::u8, Type_t::u16, Type_t::u32, Type_t::u64})
        if (Type(t).get_type_name() == name) return Type(t);
    throw Exception("unknown element type '" + name + "'");
}
}  // namespace element

// ------------------------------------------------------------------------------ shapes
class Shape : public std::vector<size_t> {
public:
    using std::vector<size_t>::vector;
    Shape() = default;
    Shape(const std::vector<size_t>& v) : std::vector<size_t>(v) {}
    std::string to_string() const {
        std::string r = "[";
        for (size_t i = 0; i < size(); i++) r += (i ? "," : "") + std::to_string((*this)[i]);
        return r + "]";
    }
};
inline std::ostream& operator<<(std::ostream& os, const Shape& s) { return os << s.to_string(); }
inline size_t shape_size(const Shape& s) {
    size_t n = 1;
    for (size_t d : s) n *= d;
    return n;
}
using Strides = std::vector<size_t>;

class Dimension {
public:
    Dimension() = default;  // dynamic
    Dimension(int64_t v) : v_(v < 0 ? -1 : v) {}
    static Dimension dynamic() { return Dimension(); }
    bool is_static() const { return v_ >= 0; }
    bool is_dynamic() const { return v_ < 0; }
    int64_t get_length() const {
        if (v_ < 0) throw Exception("Cannot get length of dynamic dimension");
        return v_;
    }
    bool compatible(const Dimension& o) const { return v_ < 0 || o.v_ < 0 || v_ == o.v_; }
    friend bool operator==(const Dimension& a, const Dimension& b) { return a.v_ == b.v_; }
    friend bool operator!=(const Dimension& a, const Dimension& b) { return a.v_ != b.v_; }

private:
    int64_t v_ = -1;
};
inline std::ostream& operator<<(std::ostream& os, const Dimension& d) {
    return d.is_static() ? os << d.get_length() : os << "?";
}

class PartialShape {
public:
    PartialShape() = default;  // rank 0
    PartialShape(std::initializer_list<Dimension> dims) : dims_(dims) {}
    PartialShape(std::vector<Dimension> dims) : dims_(std::move(dims)) {}
    PartialShape(const Shape& s) {
        for (size_t d : s) dims_.emplace_back((int64_t)d);
    }
    Dimension rank() const { return Dimension((int64_t)dims_.size()); }
    size_t size() const { return dims_.size(); }
    const Dimension& operator[](size_t i) const { return dims_.at(i); }
    Dimension& operator[](size_t i) { return dims_.at(i); }
    bool is_static() const {
        return std::all_of(dims_.begin(), dims_.end(), [](const Dimension& d) { return d.is_static(); });
    }
    bool is_dynamic() const { return !is_static(); }
    Shape to_shape() const {
        Shape s;
        for (const auto& d : dims_) s.push_back((size_t)d.get_length());
        return s;
    }
    Shape get_shape() const { return to_shape(); }
    bool compatible(const PartialShape& o) const {
        if (dims_.size() != o.dims_.size()) return false;
        for (size_t i = 0; i < dims_.size(); i++)
            if (!dims_[i].compatible(o.dims_[i])) return false;
        return true;
    }
    std::vector<Dimension>::const_iterator begin() const { return dims_.begin(); }
    std::vector<Dimension>::const_iterator end() const { return dims_.end(); }
    friend bool operator==(const PartialShape& a, const PartialShape& b) { return a.dims_ == b.dims_; }
    std::string to_string() const {
        std::ostringstream ss;
        ss << "[";
        for (size_t i = 0; i < dims_.size(); i++) ss << (i ? "," : "") << dims_[i];
        ss << "]";
        return ss.str();
    }

private:
    std::vector<Dimension> dims_;
};
inline std::ostream& operator<<(std::ostream& os, const PartialShape& s) { return os << s.to_string(); }

// ------------------------------------------------------------------------------ graph
struct DiscreteTypeInfo {
    const char* name;
    const char* version_id;
    bool operator==(const DiscreteTypeInfo& o) const {
        return std::strcmp(name, o.name) == 0 && std::strcmp(version_id, o.version_id) == 0;
    }
};

class Node;
template <typename T>
class Output;

template <>
class Output<Node> {
public:
    Output() = default;
    Output(const std::shared_ptr<Node>& node, size_t index = 0) : node_(node), index_(index) {}
    template <typename T, typename = std::enable_if_t<std::is_base_of_v<Node, T>>>
    Output(const std::shared_ptr<T>& node) : node_(node), index_(0) {}
    Node* get_node() const { return node_.get(); }
    std::shared_ptr<Node> get_node_shared_ptr() const { return node_; }
    size_t get_index() const { return index_; }
    inline const element::Type& get_element_type() const;
    inline const PartialShape& get_partial_shape() const;
    inline Shape get_shape() const;
    inline std::string get_any_name() const;
    inline const std::unordered_set<std::string>& get_names() const;
    inline void set_names(const std::unordered_set<std::string>& names);
    bool operator==(const Output& o) const { return node_ == o.node_ && index_ == o.index_; }
    bool operator<(const Output& o) const { return node_ < o.node_ || (node_ == o.node_ && index_ < o.index_); }

private:
    std::shared_ptr<Node> node_;
    size_t index_ = 0;
};

template <>
class Output<const Node> {
public:
    Output() = default;
    Output(const std::shared_ptr<const Node>& node, size_t index = 0) : node_(node), index_(index) {}
    Output(const Output<Node>& o) : node_(o.get_node_shared_ptr()), index_(o.get_index()) {}
    const Node* get_node() const { return node_.get(); }
    std::shared_ptr<const Node> get_node_shared_ptr() const { return node_; }
    size_t get_index() const { return index_; }
    inline const element::Type& get_element_type() const;
    inline const PartialShape& get_partial_shape() const;
    inline Shape get_shape() const;
    inline std::string get_any_name() const;
    inline const std::unordered_set<std::string>& get_names() const;
    bool operator==(const Output& o) const { return node_ == o.node_ && index_ == o.index_; }
    bool operator<(const Output& o) const { return node_ < o.node_ || (node_ == o.node_ && index_ < o.index_); }

private:
    std::shared_ptr<const Node> node_;
    size_t index_ = 0;
};
using OutputVector = std::vector<Output<Node>>;

class Node : public std::enable_shared_from_this<Node> {
public:
    using RTMap = std::map<std::string, Any>;
    virtual ~Node() = default;
    virtual const DiscreteTypeInfo& get_type_info() const = 0;
    const char* get_type_name() const { return get_type_info().name; }
    const std::string& get_friendly_name() const { return friendly_name_.empty() ? unique_name_ : friendly_name_; }
    void set_friendly_name(const std::string& name) { friendly_name_ = name; }
    const std::string& get_name() const { return unique_name_; }
    size_t get_input_size() const { return inputs_.size(); }
    size_t get_output_size() const { return out_types_.size(); }
    Output<Node> input_value(size_t i) const { return inputs_.at(i); }
    std::shared_ptr<Node> get_input_node_shared_ptr(size_t i) const { return inputs_.at(i).get_node_shared_ptr(); }
    OutputVector input_values() const { return inputs_; }
    Output<Node> output(size_t i) { return Output<Node>(shared_from_this(), i); }
    Output<const Node> output(size_t i) const { return Output<const Node>(shared_from_this(), i); }
    const element::Type& get_input_element_type(size_t i) const {
        const auto& in = inputs_.at(i);
        return in.get_node()->get_output_element_type(in.get_index());
    }
    const PartialShape& get_input_partial_shape(size_t i) const {
        const auto& in = inputs_.at(i);
        return in.get_node()->get_output_partial_shape(in.get_index());
    }
    const element::Type& get_output_element_type(size_t i) const { return out_types_.at(i); }
    const PartialShape& get_output_partial_shape(size_t i) const { return out_shapes_.at(i); }
    const element::Type& get_element_type() const { return out_types_.at(0); }
    Shape get_input_shape(size_t i) const { return get_input_partial_shape(i).to_shape(); }
    Shape get_output_shape(size_t i) const { return out_shapes_.at(i).to_shape(); }
    bool is_dynamic() const {
        for (size_t i = 0; i < inputs_.size(); i++)
            if (get_input_partial_shape(i).is_dynamic()) return true;
        for (const auto& s : out_shapes_)
            if (s.is_dynamic()) return true;
        return false;
    }
    RTMap& get_rt_info() { return rt_info_; }
    const RTMap& get_rt_info() const { return rt_info_; }
    // per-port tensor names
    std::unordered_set<std::string>& output_names(size_t i) { return out_names_.at(i); }
    const std::unordered_set<std::string>& output_names(size_t i) const { return out_names_.at(i); }
    void set_output_type(size_t i, const element::Type& type, const PartialShape& shape) {
        if (out_types_.size() <= i) {
            out_types_.resize(i + 1);
            out_shapes_.resize(i + 1);
            out_names_.resize(i + 1);
        }
        out_types_[i] = type;
        out_shapes_[i] = shape;
    }
    virtual void validate_and_infer_types() {}
    // attributes as text, for the stand-in serialisation
    virtual std::map<std::string, std::string> standin_attributes() const { return {}; }

protected:
    Node() : unique_name_("node_" + std::to_string(next_id()++)) {}
    explicit Node(const OutputVector& inputs) : Node() { inputs_ = inputs; }
    void set_arguments(const OutputVector& inputs) { inputs_ = inputs; }
    void constructor_validate_and_infer_types() { validate_and_infer_types(); }

private:
    static std::atomic<size_t>& next_id() {
        static std::atomic<size_t> id{0};
        return id;
    }
    std::string unique_name_, friendly_name_;
    OutputVector inputs_;
    std::vector<element::Type> out_types_;
    std::vector<PartialShape> out_shapes_;
    std::vector<std::unordered_set<std::string>> out_names_;
    RTMap rt_info_;
};

inline const element::Type& Output<Node>::get_element_type() const { return node_->get_output_element_type(index_); }
inline const PartialShape& Output<Node>::get_partial_shape() const { return node_->get_output_partial_shape(index_); }
inline Shape Output<Node>::get_shape() const { return get_partial_shape().to_shape(); }
inline const std::unordered_set<std::string>& Output<Node>::get_names() const { return node_->output_names(index_); }
inline void Output<Node>::set_names(const std::unordered_set<std::string>& names) { node_->output_names(index_) = names; }
inline std::string Output<Node>::get_any_name() const {
    const auto& names = get_names();
    if (names.empty()) throw Exception("Attempt to get a name for a Tensor without names");
    return *std::min_element(names.begin(), names.end());
}
inline const element::Type& Output<const Node>::get_element_type() const { return node_->get_output_element_type(index_); }
inline const PartialShape& Output<const Node>::get_partial_shape() const { return node_->get_output_partial_shape(index_); }
inline Shape Output<const Node>::get_shape() const { return get_partial_shape().to_shape(); }
inline const std::unordered_set<std::string>& Output<const Node>::get_names() const { return node_->output_names(index_); }
inline std::string Output<const Node>::get_any_name() const {
    const auto& names = get_names();
    if (names.empty()) throw Exception("Attempt to get a name for a Tensor without names");
    return *std::min_element(names.begin(), names.end());
}

template <typename T, typename U>
std::shared_ptr<T> as_type_ptr(const std::shared_ptr<U>& p) {
    return std::dynamic_pointer_cast<T>(p);
}
template <typename T, typename U>
T* as_type(U* p) {
    return dynamic_cast<T*>(p);
}
template <typename T, typename U>
bool is_type(const std::shared_ptr<U>& p) {
    return std::dynamic_pointer_cast<T>(p) != nullptr;
}

#define OPENVINO_OP(NAME, VERSION)                                      \
    const ::ov::DiscreteTypeInfo& get_type_info() const override {      \
        static const ::ov::DiscreteTypeInfo info{NAME, VERSION};        \
        return info;                                                    \
    }

namespace op {
namespace util {
struct VariableInfo {
    PartialShape data_shape;
    element::Type data_type;
    std::string variable_id;
};
class Variable {
public:
    explicit Variable(const VariableInfo& info) : info_(info) {}
    const VariableInfo& get_info() const { return info_; }

private:
    VariableInfo info_;
};
using VariableVector = std::vector<std::shared_ptr<Variable>>;
class VariableExtension {
public:
    virtual ~VariableExtension() = default;
    std::shared_ptr<Variable> get_variable() const { return variable_; }
    virtual std::string get_variable_id() const { return variable_->get_info().variable_id; }

protected:
    std::shared_ptr<Variable> variable_;
};
class ReadValueBase : public Node, public VariableExtension {
protected:
    using Node::Node;
};
class AssignBase : public Node, public VariableExtension {  // a Sink
protected:
    using Node::Node;
};
}  // namespace util
using Sink = util::AssignBase;

namespace v0 {
class Parameter : public Node {
public:
    OPENVINO_OP("Parameter", "opset1")
    Parameter(const element::Type& type, const PartialShape& shape) { set_output_type(0, type, shape); }
    std::map<std::string, std::string> standin_attributes() const override {
        return {{"element_type", get_output_element_type(0).get_type_name()}, {"shape", get_output_partial_shape(0).to_string()}};
    }
};
class Result : public Node {
public:
    OPENVINO_OP("Result", "opset1")
    explicit Result(const Output<Node>& arg) : Node(OutputVector{arg}) {
        set_output_type(0, arg.get_element_type(), arg.get_partial_shape());
    }
};
class Constant : public Node {
public:
    OPENVINO_OP("Constant", "opset1")
    Constant(const element::Type& type, const Shape& shape, const void* data) : bytes_(type.size() * shape_size(shape)) {
        set_output_type(0, type, PartialShape(shape));
        if (!bytes_.empty()) std::memcpy(bytes_.data(), data, bytes_.size());
    }
    const void* get_data_ptr() const { return bytes_.data(); }
    size_t get_byte_size() const { return bytes_.size(); }
    // the values as T, for the integer constants that carry shapes, axes and orders
    template <typename T>
    std::vector<T> cast_vector() const {
        const element::Type& t = get_output_element_type(0);
        const size_t n = t.size() ? bytes_.size() / t.size() : 0;
        std::vector<T> out(n);
        for (size_t i = 0; i < n; i++) {
            const uint8_t* at = bytes_.data() + i * t.size();
            if (t == element::i64) { int64_t v; std::memcpy(&v, at, 8); out[i] = (T)v; }
            else if (t == element::i32) { int32_t v; std::memcpy(&v, at, 4); out[i] = (T)v; }
            else if (t == element::u64) { uint64_t v; std::memcpy(&v, at, 8); out[i] = (T)v; }
            else if (t == element::u32) { uint32_t v; std::memcpy(&v, at, 4); out[i] = (T)v; }
            else if (t == element::i8) { int8_t v; std::memcpy(&v, at, 1); out[i] = (T)v; }
            else if (t == element::u8 || t == element::boolean) { out[i] = (T)*at; }
            else if (t == element::f32) { float v; std::memcpy(&v, at, 4); out[i] = (T)v; }
            else OPENVINO_THROW("Constant::cast_vector: element type ", t.get_type_name());
        }
        return out;
    }
    std::map<std::string, std::string> standin_attributes() const override {
        std::string hex;
        static const char* digits = "0123456789abcdef";
        for (uint8_t b : bytes_) {
            hex += digits[b >> 4];
            hex += digits[b & 15];
        }
        return {{"element_type", get_output_element_type(0).get_type_name()},
                {"shape", get_output_partial_shape(0).to_string()},
                {"data", hex}};
    }

private:
    std::vector<uint8_t> bytes_;
};
}  // namespace v0

namespace v13 {
// query, key, value [, attention_mask [, scale]]; out like query
class ScaledDotProductAttention : public Node {
public:
    OPENVINO_OP("ScaledDotProductAttention", "opset13")
    ScaledDotProductAttention(const OutputVector& inputs, bool causal) : Node(inputs), causal_(causal) { infer(); }
    ScaledDotProductAttention(const Output<Node>& q, const Output<Node>& k, const Output<Node>& v, bool causal)
        : ScaledDotProductAttention(OutputVector{q, k, v}, causal) {}
    ScaledDotProductAttention(const Output<Node>& q, const Output<Node>& k, const Output<Node>& v,
                              const Output<Node>& mask, bool causal)
        : ScaledDotProductAttention(OutputVector{q, k, v, mask}, causal) {}
    ScaledDotProductAttention(const Output<Node>& q, const Output<Node>& k, const Output<Node>& v,
                              const Output<Node>& mask, const Output<Node>& scale, bool causal)
        : ScaledDotProductAttention(OutputVector{q, k, v, mask, scale}, causal) {}
    bool get_causal() const { return causal_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"causal", causal_ ? "true" : "false"}}; }

private:
    void infer() {
        OPENVINO_ASSERT(get_input_size() >= 3 && get_input_size() <= 5, "ScaledDotProductAttention takes 3 to 5 inputs");
        set_output_type(0, get_input_element_type(0), get_input_partial_shape(0));
    }
    bool causal_;
};
}  // namespace v13

// PagedAttentionExtension: 13 to 20 inputs in the operator's order; out0 like query, out1 scores
class PagedAttentionExtension : public Node {
public:
    OPENVINO_OP("PagedAttentionExtension", "extension")
    explicit PagedAttentionExtension(const OutputVector& inputs) : Node(inputs) {
        OPENVINO_ASSERT(inputs.size() >= 13, "PagedAttentionExtension takes at least 13 inputs");
        set_output_type(0, get_input_element_type(0), get_input_partial_shape(0));
        set_output_type(1, get_input_element_type(0), PartialShape{Dimension::dynamic()});
    }
    // the operator lets a transformation pin the type of an output
    void set_out_type(int index, const element::Type& type) { set_output_type((size_t)index, type, get_output_partial_shape(index)); }
    std::map<std::string, std::string> standin_attributes() const override {
        return {{"out0_type", get_output_element_type(0).get_type_name()}, {"out1_type", get_output_element_type(1).get_type_name()}};
    }
};

namespace v6 {
class ReadValue : public util::ReadValueBase {
public:
    OPENVINO_OP("ReadValue", "opset6")
    explicit ReadValue(const std::shared_ptr<util::Variable>& variable) {  // no initial value
        variable_ = variable;
        set_output_type(0, variable->get_info().data_type, variable->get_info().data_shape);
    }
    ReadValue(const Output<Node>& init_value, const std::shared_ptr<util::Variable>& variable)
        : util::ReadValueBase(OutputVector{init_value}) {
        variable_ = variable;
        set_output_type(0, variable->get_info().data_type, variable->get_info().data_shape);
    }
    std::map<std::string, std::string> standin_attributes() const override { return {{"variable_id", get_variable_id()}}; }
};
class Assign : public util::AssignBase {
public:
    OPENVINO_OP("Assign", "opset6")
    Assign(const Output<Node>& new_value, const std::shared_ptr<util::Variable>& variable)
        : util::AssignBase(OutputVector{new_value}) {
        variable_ = variable;
        set_output_type(0, new_value.get_element_type(), new_value.get_partial_shape());
    }
    std::map<std::string, std::string> standin_attributes() const override { return {{"variable_id", get_variable_id()}}; }
};
}  // namespace v6

namespace util {
// numpy's broadcasting rule on shapes that may hold unknown extents
inline PartialShape broadcast_shapes(const PartialShape& a, const PartialShape& b) {
    const size_t rank = std::max(a.size(), b.size());
    std::vector<Dimension> dims(rank);
    for (size_t k = 0; k < rank; k++) {
        const Dimension da = k + a.size() >= rank ? a[k + a.size() - rank] : Dimension(1);
        const Dimension db = k + b.size() >= rank ? b[k + b.size() - rank] : Dimension(1);
        if (da.is_static() && db.is_static()) {
            OPENVINO_ASSERT(da.get_length() == db.get_length() || da.get_length() == 1 || db.get_length() == 1,
                            "shapes ", a.to_string(), " and ", b.to_string(), " do not broadcast");
            dims[k] = da.get_length() == 1 ? db : da;
        } else if (da.is_static() && da.get_length() != 1) {
            dims[k] = da;
        } else if (db.is_static() && db.get_length() != 1) {
            dims[k] = db;
        } else {
            dims[k] = Dimension::dynamic();
        }
    }
    return PartialShape(dims);
}
// element-wise arithmetic of two tensors under numpy broadcasting
class BinaryElementwiseArithmetic : public Node {
protected:
    BinaryElementwiseArithmetic(const Output<Node>& a, const Output<Node>& b) : Node(OutputVector{a, b}) {
        set_output_type(0, a.get_element_type(), broadcast_shapes(a.get_partial_shape(), b.get_partial_shape()));
    }
};
}  // namespace util

namespace v1 {
class Add : public util::BinaryElementwiseArithmetic {
public:
    OPENVINO_OP("Add", "opset1")
    Add(const Output<Node>& a, const Output<Node>& b) : util::BinaryElementwiseArithmetic(a, b) {}
};
class Subtract : public util::BinaryElementwiseArithmetic {
public:
    OPENVINO_OP("Subtract", "opset1")
    Subtract(const Output<Node>& a, const Output<Node>& b) : util::BinaryElementwiseArithmetic(a, b) {}
};
class Divide : public util::BinaryElementwiseArithmetic {
public:
    OPENVINO_OP("Divide", "opset1")
    Divide(const Output<Node>& a, const Output<Node>& b) : util::BinaryElementwiseArithmetic(a, b) {}
};
// exp(x - max) / sum over one axis
class Softmax : public Node {
public:
    OPENVINO_OP("Softmax", "opset1")
    Softmax(const Output<Node>& x, size_t axis) : Node(OutputVector{x}), axis_(axis) {
        set_output_type(0, x.get_element_type(), x.get_partial_shape());
    }
    size_t get_axis() const { return axis_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"axis", std::to_string(axis_)}, {"opset", "1"}}; }

private:
    size_t axis_;
};
}  // namespace v1

namespace v8 {
// as v1, the axis may count from the end
class Softmax : public Node {
public:
    OPENVINO_OP("Softmax", "opset8")
    Softmax(const Output<Node>& x, int64_t axis) : Node(OutputVector{x}), axis_(axis) {
        set_output_type(0, x.get_element_type(), x.get_partial_shape());
    }
    int64_t get_axis() const { return axis_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"axis", std::to_string(axis_)}, {"opset", "8"}}; }

private:
    int64_t axis_;
};
}  // namespace v8

namespace v0 {
// A [.., m, k] x B [.., k, n] with optional transposition of the last two axes of either operand
class MatMul : public Node {
public:
    OPENVINO_OP("MatMul", "opset1")
    MatMul(const Output<Node>& a, const Output<Node>& b, bool transpose_a = false, bool transpose_b = false)
        : Node(OutputVector{a, b}), transpose_a_(transpose_a), transpose_b_(transpose_b) {
        const PartialShape &sa = a.get_partial_shape(), &sb = b.get_partial_shape();
        OPENVINO_ASSERT(sa.size() >= 2 && sb.size() >= 2, "MatMul operands must have rank 2 or more");
        const PartialShape& lead = sa.size() >= sb.size() ? sa : sb;
        std::vector<Dimension> dims(lead.begin(), lead.end() - 2);
        dims.push_back(sa[sa.size() - (transpose_a ? 1 : 2)]);
        dims.push_back(sb[sb.size() - (transpose_b ? 2 : 1)]);
        set_output_type(0, a.get_element_type(), PartialShape(dims));
    }
    bool get_transpose_a() const { return transpose_a_; }
    bool get_transpose_b() const { return transpose_b_; }
    std::map<std::string, std::string> standin_attributes() const override {
        return {{"transpose_a", transpose_a_ ? "true" : "false"}, {"transpose_b", transpose_b_ ? "true" : "false"}};
    }

private:
    bool transpose_a_, transpose_b_;
};

class Concat : public Node {
public:
    OPENVINO_OP("Concat", "opset1")
    Concat(const OutputVector& args, int64_t axis) : Node(args), axis_(axis) {
        OPENVINO_ASSERT(!args.empty(), "Concat without inputs");
        PartialShape out = args[0].get_partial_shape();
        const int64_t ax = axis < 0 ? axis + (int64_t)out.size() : axis;
        OPENVINO_ASSERT(ax >= 0 && ax < (int64_t)out.size(), "Concat axis out of range");
        std::vector<Dimension> dims(out.begin(), out.end());
        bool dynamic = false;
        int64_t total = 0;
        for (const auto& a : args) {
            const auto& d = a.get_partial_shape()[ax];
            if (d.is_dynamic())
                dynamic = true;
            else
                total += d.get_length();
        }
        dims[ax] = dynamic ? Dimension::dynamic() : Dimension(total);
        set_output_type(0, args[0].get_element_type(), PartialShape(dims));
    }
    int64_t get_axis() const { return axis_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"axis", std::to_string(axis_)}}; }

private:
    int64_t axis_;
};
}  // namespace v0

namespace util {
// data, indices, axis (a Constant); batch_dims as attribute
class GatherBase : public Node {
public:
    int64_t get_axis() const {
        auto c = std::dynamic_pointer_cast<v0::Constant>(get_input_node_shared_ptr(2));
        OPENVINO_ASSERT(c && c->get_byte_size() >= 4, "Gather axis must be a constant");
        int64_t axis = 0;
        if (c->get_output_element_type(0).size() == 8)
            std::memcpy(&axis, c->get_data_ptr(), 8);
        else {
            int32_t a32;
            std::memcpy(&a32, c->get_data_ptr(), 4);
            axis = a32;
        }
        return axis < 0 ? axis + (int64_t)get_input_partial_shape(0).size() : axis;
    }
    int64_t get_batch_dims() const { return batch_dims_; }

protected:
    GatherBase(const Output<Node>& data, const Output<Node>& indices, const Output<Node>& axis, int64_t batch_dims)
        : Node(OutputVector{data, indices, axis}), batch_dims_(batch_dims) {
        const PartialShape &d = data.get_partial_shape(), &i = indices.get_partial_shape();
        const int64_t ax = get_axis();
        OPENVINO_ASSERT(ax >= 0 && ax < (int64_t)d.size() && batch_dims >= 0 && batch_dims <= ax, "Gather axis / batch_dims out of range");
        std::vector<Dimension> dims(d.begin(), d.begin() + ax);
        dims.insert(dims.end(), i.begin() + batch_dims, i.end());
        dims.insert(dims.end(), d.begin() + ax + 1, d.end());
        set_output_type(0, data.get_element_type(), PartialShape(dims));
    }
    int64_t batch_dims_;
};
}  // namespace util

namespace v8 {
class Gather : public util::GatherBase {
public:
    OPENVINO_OP("Gather", "opset8")
    Gather(const Output<Node>& data, const Output<Node>& indices, const Output<Node>& axis, int64_t batch_dims = 0)
        : util::GatherBase(data, indices, axis, batch_dims) {}
    std::map<std::string, std::string> standin_attributes() const override {
        return {{"batch_dims", std::to_string(batch_dims_)}};
    }
};
}  // namespace v8

namespace util {
// the integer values of a Constant input, or nothing when the input is computed at run time
inline bool constant_values(const Output<Node>& input, std::vector<int64_t>& values) {
    auto c = std::dynamic_pointer_cast<v0::Constant>(input.get_node_shared_ptr());
    if (!c) return false;
    values = c->cast_vector<int64_t>();
    return true;
}
}  // namespace util

namespace v1 {
// data, pattern: the same elements under the extents of `pattern`; -1 takes what is left, 0 copies
// the input's extent at that position when special_zero is set
class Reshape : public Node {
public:
    OPENVINO_OP("Reshape", "opset1")
    Reshape(const Output<Node>& data, const Output<Node>& pattern, bool special_zero)
        : Node(OutputVector{data, pattern}), special_zero_(special_zero) {
        std::vector<int64_t> want;
        const PartialShape& in = data.get_partial_shape();
        if (util::constant_values(pattern, want)) {
            std::vector<Dimension> dims;
            for (size_t i = 0; i < want.size(); i++) {
                if (want[i] == 0 && special_zero && i < in.size())
                    dims.push_back(in[i]);
                else if (want[i] < 0)
                    dims.push_back(Dimension::dynamic());
                else
                    dims.push_back(Dimension(want[i]));
            }
            if (in.is_static()) {  // the one -1 can be settled now
                int64_t known = 1, total = (int64_t)shape_size(in.to_shape());
                int open = -1;
                for (size_t i = 0; i < dims.size(); i++) {
                    if (dims[i].is_dynamic())
                        open = (int)i;
                    else
                        known *= dims[i].get_length();
                }
                if (open >= 0 && known > 0) dims[open] = Dimension(total / known);
            }
            set_output_type(0, data.get_element_type(), PartialShape(dims));
        } else {
            const PartialShape& ps = pattern.get_partial_shape();
            OPENVINO_ASSERT(ps.size() == 1 && ps[0].is_static(), "Reshape pattern must be a vector of known length");
            set_output_type(0, data.get_element_type(), PartialShape(std::vector<Dimension>((size_t)ps[0].get_length(), Dimension::dynamic())));
        }
    }
    bool get_special_zero() const { return special_zero_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"special_zero", special_zero_ ? "true" : "false"}}; }

private:
    bool special_zero_;
};

// data, order: output axis k is input axis order[k]; an empty order reverses the axes
class Transpose : public Node {
public:
    OPENVINO_OP("Transpose", "opset1")
    Transpose(const Output<Node>& data, const Output<Node>& order) : Node(OutputVector{data, order}) {
        const PartialShape& in = data.get_partial_shape();
        std::vector<int64_t> perm;
        std::vector<Dimension> dims(in.size(), Dimension::dynamic());
        if (util::constant_values(order, perm)) {
            if (perm.empty())
                for (size_t k = 0; k < in.size(); k++) perm.push_back((int64_t)(in.size() - 1 - k));
            OPENVINO_ASSERT(perm.size() == in.size(), "Transpose order must name every axis");
            for (size_t k = 0; k < perm.size(); k++) {
                OPENVINO_ASSERT(perm[k] >= 0 && perm[k] < (int64_t)in.size(), "Transpose order out of range");
                dims[k] = in[(size_t)perm[k]];
            }
        }
        set_output_type(0, data.get_element_type(), PartialShape(dims));
    }
};
}  // namespace v1

namespace v0 {
// data [, axes]: axes of extent 1 removed (all of them without the second input)
class Squeeze : public Node {
public:
    OPENVINO_OP("Squeeze", "opset1")
    explicit Squeeze(const OutputVector& args) : Node(args) {
        OPENVINO_ASSERT(args.size() == 1 || args.size() == 2, "Squeeze takes data [, axes]");
        const PartialShape& in = args[0].get_partial_shape();
        std::vector<int64_t> axes;
        const bool known = args.size() == 1 || util::constant_values(args[1], axes);
        OPENVINO_ASSERT(known, "Squeeze axes must be a Constant");
        std::vector<bool> drop(in.size(), false);
        for (int64_t a : axes) {
            if (a < 0) a += (int64_t)in.size();
            OPENVINO_ASSERT(a >= 0 && a < (int64_t)in.size(), "Squeeze axis out of range");
            drop[(size_t)a] = true;
        }
        std::vector<Dimension> dims;
        for (size_t k = 0; k < in.size(); k++) {
            const bool one = in[k].is_static() && in[k].get_length() == 1;
            if (args.size() == 1 ? one : (drop[k] && (one || in[k].is_dynamic()))) continue;
            dims.push_back(in[k]);
        }
        set_output_type(0, args[0].get_element_type(), PartialShape(dims));
    }
};

// data, axes: axes of extent 1 inserted at the given positions of the output
class Unsqueeze : public Node {
public:
    OPENVINO_OP("Unsqueeze", "opset1")
    Unsqueeze(const Output<Node>& data, const Output<Node>& axes_input) : Node(OutputVector{data, axes_input}) {
        const PartialShape& in = data.get_partial_shape();
        std::vector<int64_t> axes;
        OPENVINO_ASSERT(util::constant_values(axes_input, axes), "Unsqueeze axes must be a Constant");
        const int64_t rank = (int64_t)(in.size() + axes.size());
        std::vector<bool> fresh((size_t)rank, false);
        for (int64_t a : axes) {
            if (a < 0) a += rank;
            OPENVINO_ASSERT(a >= 0 && a < rank && !fresh[(size_t)a], "Unsqueeze axis out of range or repeated");
            fresh[(size_t)a] = true;
        }
        std::vector<Dimension> dims;
        for (size_t k = 0, next = 0; k < (size_t)rank; k++) dims.push_back(fresh[k] ? Dimension(1) : in[next++]);
        set_output_type(0, data.get_element_type(), PartialShape(dims));
    }
};

// data: the same values in another element type
class Convert : public Node {
public:
    OPENVINO_OP("Convert", "opset1")
    Convert(const Output<Node>& data, const element::Type& destination_type) : Node(OutputVector{data}), destination_(destination_type) {
        set_output_type(0, destination_type, data.get_partial_shape());
    }
    const element::Type& get_destination_type() const { return destination_; }
    const element::Type& get_convert_element_type() const { return destination_; }
    std::map<std::string, std::string> standin_attributes() const override { return {{"destination_type", destination_.get_type_name()}}; }

private:
    element::Type destination_;
};
}  // namespace v0

namespace v4 {
// x [, beta]: x / (1 + exp(-beta x))
class Swish : public Node {
public:
    OPENVINO_OP("Swish", "opset4")
    explicit Swish(const OutputVector& args) : Node(args) {
        OPENVINO_ASSERT(args.size() == 1 || args.size() == 2, "Swish takes x [, beta]");
        set_output_type(0, args[0].get_element_type(), args[0].get_partial_shape());
    }
};
}  // namespace v4

namespace v1 {
class Multiply : public util::BinaryElementwiseArithmetic {
public:
    OPENVINO_OP("Multiply", "opset1")
    Multiply(const Output<Node>& a, const Output<Node>& b) : util::BinaryElementwiseArithmetic(a, b) {}
};
}  // namespace v1

namespace internal {
// data split in two along `axis` (split_lengths wide each): act(half split_to_glu_idx) * other half
class GLU : public Node {
public:
    OPENVINO_OP("GLU", "ie_internal_opset")
    enum GluType { Swish = 0, Gelu, Gelu_Tanh };
    GLU(const Output<Node>& data, int64_t axis, int64_t split_lengths, const GluType glu_type, const size_t split_to_glu_idx,
        const element::Type output_type = element::dynamic)
        : Node(OutputVector{data}), axis_(axis), split_lengths_(split_lengths), glu_type_(glu_type),
          split_to_glu_idx_(split_to_glu_idx), output_type_(output_type) {
        const PartialShape& ps = data.get_partial_shape();
        std::vector<Dimension> dims(ps.begin(), ps.end());
        const int64_t ax = axis < 0 ? axis + (int64_t)dims.size() : axis;
        OPENVINO_ASSERT(ax >= 0 && ax < (int64_t)dims.size(), "GLU axis out of range");
        dims[ax] = Dimension(split_lengths);
        set_output_type(0, output_type == element::dynamic ? data.get_element_type() : output_type, PartialShape(dims));
    }
    int64_t get_axis() const { return axis_; }
    int64_t get_split_lengths() const { return split_lengths_; }
    GluType get_glu_type() const { return glu_type_; }
    size_t get_split_to_glu_idx() const { return split_to_glu_idx_; }
    const element::Type& get_output_type() const { return output_type_; }
    std::map<std::string, std::string> standin_attributes() const override {
        return {{"axis", std::to_string(axis_)}, {"split_lengths", std::to_string(split_lengths_)},
                {"glu_type", std::to_string((int)glu_type_)}, {"split_to_glu_idx", std::to_string(split_to_glu_idx_)},
                {"output_type", output_type_.get_type_name()}};
    }

private:
    int64_t axis_, split_lengths_;
    GluType glu_type_;
    size_t split_to_glu_idx_;
    element::Type output_type_;
};

// data, gamma; out = data / sqrt(mean(data^2, last axis) + epsilon) * gamma
class RMS : public Node {
public:
    OPENVINO_OP("RMS", "ie_internal_opset")
    RMS(const Output<Node>& data, const Output<Node>& gamma, double epsilon, const element::Type output_type = element::dynamic)
        : Node(OutputVector{data, gamma}), epsilon_(epsilon), output_type_(output_type) {
        set_output_type(0, output_type == element::dynamic ? data.get_element_type() : output_type, data.get_partial_shape());
    }
    double get_epsilon() const { return epsilon_; }
    const element::Type& get_output_type() const { return output_type_; }
    std::map<std::string, std::string> standin_attributes() const override {
        std::ostringstream e;
        e.precision(17);
        e << epsilon_;
        return {{"epsilon", e.str()}, {"output_type", output_type_.get_type_name()}};
    }

private:
    double epsilon_;
    element::Type output_type_;
};

// x, cos, sin [, position ids]; rotary position embedding with the layout described by Config
class RoPE : public Node {
public:
    OPENVINO_OP("RoPE", "ie_internal_opset")
    struct Config {
        size_t slice_start = 0;  // slice of the innermost axis of x that holds the heads to rotate
        size_t slice_stop = 0;
        bool input_trans0213 = false;   // x comes as [batch, length, heads, size] instead of [batch, heads, length, size]
        bool output_trans0213 = false;  // the output is wanted as [batch, length, heads, size]
        bool is_interleaved = false;    // adjacent pairs instead of rotate-half
        size_t rotary_ndims = 0;
        bool is_chatglm = false;
        bool support_2d_rope = false;
        bool is_qwen = false;
        bool use_rope_cache = false;
        size_t head_cnt = 0;
        size_t head_size = 0;
        int gather_position_arg_id = 0;  // index of the position input, 0 = none
    };
    RoPE(const OutputVector& args, const Config& cfg) : Node(args), config_(cfg) {
        OPENVINO_ASSERT(args.size() >= 3, "RoPE takes x, cos, sin [, positions]");
        const PartialShape& x = args[0].get_partial_shape();
        std::vector<Dimension> dims(x.begin(), x.end());
        if (dims.size() == 2 && cfg.head_cnt && cfg.head_size) {  // [tokens, packed] -> [tokens, heads * size]
            dims[1] = Dimension((int64_t)(cfg.head_cnt * cfg.head_size));
        } else if (dims.size() == 3 && cfg.head_cnt && cfg.head_size) {  // [batch, length, packed] -> heads split out
            dims[2] = Dimension((int64_t)cfg.head_cnt);
            dims.push_back(Dimension((int64_t)cfg.head_size));
            if (!cfg.output_trans0213) std::swap(dims[1], dims[2]);
        } else if (dims.size() == 4 && cfg.input_trans0213 != cfg.output_trans0213) {
            std::swap(dims[1], dims[2]);
        }
        set_output_type(0, args[0].get_element_type(), PartialShape(dims));
    }
    const Config& get_config() const { return config_; }
    std::map<std::string, std::string> standin_attributes() const override {
        auto b = [](bool v) { return std::string(v ? "true" : "false"); };
        return {{"slice_start", std::to_string(config_.slice_start)}, {"slice_stop", std::to_string(config_.slice_stop)},
                {"input_trans0213", b(config_.input_trans0213)}, {"output_trans0213", b(config_.output_trans0213)},
                {"is_interleaved", b(config_.is_interleaved)}, {"rotary_ndims", std::to_string(config_.rotary_ndims)},
                {"is_chatglm", b(config_.is_chatglm)}, {"support_2d_rope", b(config_.support_2d_rope)},
                {"is_qwen", b(config_.is_qwen)}, {"use_rope_cache", b(config_.use_rope_cache)},
                {"head_cnt", std::to_string(config_.head_cnt)}, {"head_size", std::to_string(config_.head_size)},
                {"gather_position_arg_id", std::to_string(config_.gather_position_arg_id)}};
    }

private:
    Config config_;
};
}  // namespace internal
}  // namespace op

using ParameterVector = std::vector<std::shared_ptr<op::v0::Parameter>>;
using ResultVector = std::vector<std::shared_ptr<op::v0::Result>>;
using SinkVector = std::vector<std::shared_ptr<op::Sink>>;
using NodeVector = std::vector<std::shared_ptr<Node>>;

class Model : public std::enable_shared_from_this<Model> {
public:
    Model(const ResultVector& results, const ParameterVector& parameters, const std::string& name = "")
        : Model(results, SinkVector{}, parameters, name) {}
    Model(const ResultVector& results, const SinkVector& sinks, const ParameterVector& parameters,
          const std::string& name = "")
        : results_(results), sinks_(sinks), parameters_(parameters), name_(name) {
        build_order();
    }
    const std::string& get_friendly_name() const { return name_; }
    void set_friendly_name(const std::string& n) { name_ = n; }
    const std::string& get_name() const { return name_; }
    const ParameterVector& get_parameters() const { return parameters_; }
    const ResultVector& get_results() const { return results_; }
    const SinkVector& get_sinks() const { return sinks_; }
    op::util::VariableVector get_variables() const {
        op::util::VariableVector vars;
        for (const auto& n : order_)
            if (auto ext = std::dynamic_pointer_cast<op::util::VariableExtension>(n)) {
                auto v = ext->get_variable();
                if (std::find(vars.begin(), vars.end(), v) == vars.end()) vars.push_back(v);
            }
        return vars;
    }
    std::vector<std::shared_ptr<Node>> get_ordered_ops() const { return order_; }
    std::vector<std::shared_ptr<Node>> get_ops() const { return order_; }
    std::vector<Output<Node>> inputs() {
        std::vector<Output<Node>> v;
        for (auto& p : parameters_) v.emplace_back(p, 0);
        return v;
    }
    std::vector<Output<const Node>> inputs() const {
        std::vector<Output<const Node>> v;
        for (auto& p : parameters_) v.emplace_back(std::shared_ptr<const Node>(p), 0);
        return v;
    }
    std::vector<Output<Node>> outputs() {
        std::vector<Output<Node>> v;
        for (auto& r : results_) v.emplace_back(r, 0);
        return v;
    }
    std::vector<Output<const Node>> outputs() const {
        std::vector<Output<const Node>> v;
        for (auto& r : results_) v.emplace_back(std::shared_ptr<const Node>(r), 0);
        return v;
    }
    bool is_dynamic() const {
        for (auto& n : order_)
            if (n->is_dynamic()) return true;
        return false;
    }
    std::shared_ptr<Model> clone() const { return std::make_shared<Model>(results_, sinks_, parameters_, name_); }
    bool has_rt_info(const std::string& key) const { return rt_info_.count(key) != 0; }
    template <typename T>
    T get_rt_info(const std::string& key) const {
        return rt_info_.at(key).as<T>();
    }
    std::map<std::string, Any>& get_rt_info() { return rt_info_; }

private:
    void build_order() {  // depth-first post-order from results and sinks: a topological order
        std::set<Node*> seen;
        std::function<void(const std::shared_ptr<Node>&)> visit = [&](const std::shared_ptr<Node>& n) {
            if (!seen.insert(n.get()).second) return;
            for (size_t i = 0; i < n->get_input_size(); i++) visit(n->get_input_node_shared_ptr(i));
            order_.push_back(n);
        };
        for (auto& p : parameters_) visit(p);
        for (auto& r : results_) visit(r);
        for (auto& s : sinks_) visit(s);
    }
    ResultVector results_;
    SinkVector sinks_;
    ParameterVector parameters_;
    std::string name_;
    std::vector<std::shared_ptr<Node>> order_;
    std::map<std::string, Any> rt_info_;
};

// ------------------------------------------------------------------------------ tensors
template <class T>
struct SoPtr {
    SoPtr() = default;
    SoPtr(const std::shared_ptr<T>& ptr, const std::shared_ptr<void>& so = nullptr) : _ptr(ptr), _so(so) {}
    template <class U, typename = std::enable_if_t<std::is_base_of_v<T, U>>>
    SoPtr(const SoPtr<U>& o) : _ptr(o._ptr), _so(o._so) {}
    T* operator->() const noexcept { return _ptr.get(); }
    explicit operator bool() const noexcept { return _ptr != nullptr; }
    bool operator!() const noexcept { return _ptr == nullptr; }
    std::shared_ptr<T> _ptr;
    std::shared_ptr<void> _so;
};

class ITensor : public std::enable_shared_from_this<ITensor> {
public:
    virtual ~ITensor() = default;
    virtual void set_shape(Shape shape) = 0;
    virtual const element::Type& get_element_type() const = 0;
    virtual const Shape& get_shape() const = 0;
    virtual size_t get_size() const { return shape_size(get_shape()); }
    virtual size_t get_byte_size() const { return get_size() * get_element_type().size(); }
    virtual void* data(const element::Type& type = {}) const = 0;
    virtual bool is_continuous() const { return true; }
    virtual void copy_to(const std::shared_ptr<ITensor>& dst) const {
        OPENVINO_ASSERT(dst->get_element_type() == get_element_type(), "copy_to: element types differ");
        if (dst->get_shape() != get_shape()) dst->set_shape(get_shape());
        if (get_byte_size()) std::memcpy(dst->data(), data(), get_byte_size());
    }
    template <typename T>
    T* data() const {
        return static_cast<T*>(data(element::Type{}));
    }
};

class IRemoteTensor : public ITensor {
public:
    void* data(const element::Type& = {}) const override { OPENVINO_NOT_IMPLEMENTED; }
    virtual const AnyMap& get_properties() const = 0;
    virtual const std::string& get_device_name() const = 0;
};

namespace standin {
class HostTensor : public ITensor {
public:
    HostTensor(const element::Type& type, const Shape& shape, void* external = nullptr)
        : type_(type), shape_(shape), external_(external) {
        if (!external_) storage_.resize(std::max<size_t>(get_byte_size(), 1));
    }
    void set_shape(Shape shape) override {
        shape_ = std::move(shape);
        if (external_) {
            OPENVINO_ASSERT(get_byte_size() <= external_bytes_ || external_bytes_ == 0,
                            "Could set new shape: the tensor wraps preallocated memory");
        } else {
            storage_.resize(std::max<size_t>(get_byte_size(), 1));
        }
    }
    const element::Type& get_element_type() const override { return type_; }
    const Shape& get_shape() const override { return shape_; }
    void* data(const element::Type& = {}) const override { return external_ ? external_ : (void*)storage_.data(); }

private:
    element::Type type_;
    Shape shape_;
    void* external_;
    size_t external_bytes_ = 0;
    mutable std::vector<uint8_t> storage_;
};
}  // namespace standin

inline std::shared_ptr<ITensor> make_tensor(const element::Type& type, const Shape& shape) {
    return std::make_shared<standin::HostTensor>(type, shape);
}
inline std::shared_ptr<ITensor> make_tensor(const element::Type& type, const Shape& shape, void* host_ptr,
                                            const Strides& = {}) {
    return std::make_shared<standin::HostTensor>(type, shape, host_ptr);
}

// The public tensor class: a handle on an ITensor.
class Tensor {
public:
    Tensor() = default;
    Tensor(const element::Type& type, const Shape& shape) : impl_(make_tensor(type, shape)) {}
    Tensor(const element::Type& type, const Shape& shape, void* host_ptr) : impl_(make_tensor(type, shape, host_ptr)) {}
    explicit Tensor(const std::shared_ptr<ITensor>& impl) : impl_(impl) {}
    const element::Type& get_element_type() const { return impl_->get_element_type(); }
    const Shape& get_shape() const { return impl_->get_shape(); }
    void set_shape(const Shape& s) { impl_->set_shape(s); }
    size_t get_size() const { return impl_->get_size(); }
    size_t get_byte_size() const { return impl_->get_byte_size(); }
    void* data(const element::Type& t = {}) const { return impl_->data(t); }
    template <typename T>
    T* data() const {
        return static_cast<T*>(impl_->data());
    }
    explicit operator bool() const noexcept { return impl_ != nullptr; }
    const std::shared_ptr<ITensor>& standin_impl() const { return impl_; }

private:
    std::shared_ptr<ITensor> impl_;
};
inline SoPtr<ITensor> get_tensor_impl(const Tensor& t) { return SoPtr<ITensor>{t.standin_impl(), nullptr}; }
inline Tensor make_tensor(const SoPtr<ITensor>& t) { return Tensor(t._ptr); }

class IRemoteContext : public std::enable_shared_from_this<IRemoteContext> {
public:
    virtual ~IRemoteContext() = default;
    virtual const std::string& get_device_name() const = 0;
    virtual const AnyMap& get_property() const = 0;
    virtual SoPtr<IRemoteTensor> create_tensor(const element::Type& type, const Shape& shape, const AnyMap& params = {}) = 0;
    virtual SoPtr<ITensor> create_host_tensor(const element::Type type, const Shape& shape) {
        return SoPtr<ITensor>{make_tensor(type, shape), nullptr};
    }
};

class IVariableState : public std::enable_shared_from_this<IVariableState> {
public:
    explicit IVariableState(const std::string& name) : m_name(name) {}
    virtual ~IVariableState() = default;
    virtual const std::string& get_name() const { return m_name; }
    virtual void reset() = 0;
    virtual void set_state(const SoPtr<ITensor>& state) = 0;
    virtual SoPtr<ITensor> get_state() const = 0;

protected:
    std::string m_name;
    SoPtr<ITensor> m_state;
};

struct ProfilingInfo {
    enum class Status { NOT_RUN, OPTIMIZED_OUT, EXECUTED };
    Status status = Status::NOT_RUN;
    std::chrono::microseconds real_time{0};
    std::chrono::microseconds cpu_time{0};
    std::string node_name, exec_type, node_type;
};

// ------------------------------------------------------------------------------ properties
enum class PropertyMutability { RO, RW, WO };
struct PropertyName : public std::string {
    PropertyName(const std::string& s, PropertyMutability m = PropertyMutability::RW) : std::string(s), mutability(m) {}
    bool is_mutable() const { return mutability == PropertyMutability::RW; }
    PropertyMutability mutability;
};
template <typename T, PropertyMutability M = PropertyMutability::RW>
struct Property {
    constexpr explicit Property(const char* n) : n_(n) {}
    const char* name() const { return n_; }
    std::pair<std::string, Any> operator()(const T& v) const { return {n_, Any(v)}; }
    const char* n_;
};
static constexpr Property<std::vector<PropertyName>, PropertyMutability::RO> supported_properties{"SUPPORTED_PROPERTIES"};
static constexpr Property<std::vector<std::string>, PropertyMutability::RO> available_devices{"AVAILABLE_DEVICES"};
static constexpr Property<std::string, PropertyMutability::RO> model_name{"NETWORK_NAME"};
static constexpr Property<uint32_t, PropertyMutability::RO> optimal_number_of_infer_requests{"OPTIMAL_NUMBER_OF_INFER_REQUESTS"};
static constexpr Property<std::tuple<unsigned, unsigned, unsigned>, PropertyMutability::RO> range_for_async_infer_requests{
    "RANGE_FOR_ASYNC_INFER_REQUESTS"};
static constexpr Property<std::vector<std::string>, PropertyMutability::RO> execution_devices{"EXECUTION_DEVICES"};
static constexpr Property<bool, PropertyMutability::RO> loaded_from_cache{"LOADED_FROM_CACHE"};
static constexpr Property<bool> enable_profiling{"PERF_COUNT"};
static constexpr Property<int32_t> num_streams{"NUM_STREAMS"};
static constexpr Property<std::string> cache_dir{"CACHE_DIR"};
namespace device {
static constexpr Property<std::string> id{"DEVICE_ID"};
static constexpr Property<std::string, PropertyMutability::RO> full_name{"FULL_DEVICE_NAME"};
static constexpr Property<std::string, PropertyMutability::RO> architecture{"DEVICE_ARCHITECTURE"};
static constexpr Property<std::vector<std::string>, PropertyMutability::RO> capabilities{"OPTIMIZATION_CAPABILITIES"};
namespace capability {
constexpr const char* FP32 = "FP32";
constexpr const char* FP16 = "FP16";
constexpr const char* BF16 = "BF16";
constexpr const char* EXPORT_IMPORT = "EXPORT_IMPORT";
}  // namespace capability
}  // namespace device
namespace hint {
static constexpr Property<element::Type> inference_precision{"INFERENCE_PRECISION_HINT"};
enum class PerformanceMode { LATENCY = 1, THROUGHPUT = 2, CUMULATIVE_THROUGHPUT = 3 };
static constexpr Property<PerformanceMode> performance_mode{"PERFORMANCE_HINT"};
}  // namespace hint
namespace internal {
static constexpr Property<std::vector<PropertyName>, PropertyMutability::RO> supported_properties{"INTERNAL_SUPPORTED_PROPERTIES"};
static constexpr Property<std::vector<PropertyName>, PropertyMutability::RO> caching_properties{"CACHING_PROPERTIES"};
}  // namespace internal

struct Version {
    const char* buildNumber;
    const char* description;
};

// ------------------------------------------------------------------------------ executors
namespace threading {
using Task = std::function<void()>;
class ITaskExecutor {
public:
    virtual ~ITaskExecutor() = default;
    virtual void run(Task task) = 0;
    virtual void run_and_wait(const std::vector<Task>& tasks) {
        std::vector<std::future<void>> done;
        for (const auto& t : tasks) {
            auto packaged = std::make_shared<std::packaged_task<void()>>(t);
            done.push_back(packaged->get_future());
            run([packaged] { (*packaged)(); });
        }
        for (auto& f : done) f.get();
    }
};
// runs a task in the caller's thread, at once
class ImmediateExecutor : public ITaskExecutor {
public:
    void run(Task task) override { task(); }
};
}  // namespace threading

// ------------------------------------------------------------------------------ serialisation
class ICore {
public:
    virtual ~ICore() = default;
    virtual std::shared_ptr<Model> read_model(const std::string& model, const Tensor& weights, bool frontend_mode = false) const = 0;
};

namespace pass {
// Text form of a model: the part "xml" lists the nodes in topological order, one per line, as
//   <index> <type> <name> inputs=<producer index>:<port>,... {key=value;...}
// and the part "bin" is empty (constants travel in the text as hexadecimal).  Enough for the
// operators of the attention path; it stands where OpenVINO writes its IR.
class Serialize {
public:
    enum class Version : uint8_t { UNSPECIFIED = 0, IR_V10 = 10, IR_V11 = 11 };
    Serialize(std::ostream& xml, std::ostream& bin, Version = Version::UNSPECIFIED) : xml_(xml), bin_(bin) {}
    bool run_on_model(const std::shared_ptr<Model>& model) {
        std::map<const Node*, size_t> index;
        xml_ << "standin-ir 1 " << model->get_friendly_name() << "\n";
        const auto ops = model->get_ordered_ops();
        for (size_t i = 0; i < ops.size(); i++) {
            const auto& n = ops[i];
            index[n.get()] = i;
            xml_ << i << " " << n->get_type_info().name << " " << n->get_friendly_name() << " inputs=";
            for (size_t k = 0; k < n->get_input_size(); k++) {
                const auto in = n->input_value(k);
                xml_ << (k ? "," : "") << index.at(in.get_node()) << ":" << in.get_index();
            }
            xml_ << " {";
            for (const auto& [key, value] : n->standin_attributes()) xml_ << key << "=" << value << ";";
            if (auto ext = std::dynamic_pointer_cast<op::util::VariableExtension>(n)) {
                const auto& info = ext->get_variable()->get_info();
                xml_ << "variable_type=" << info.data_type.get_type_name() << ";variable_shape=" << info.data_shape.to_string() << ";";
            }
            xml_ << "}\n";
        }
        (void)bin_;
        return false;
    }

private:
    std::ostream& xml_;
    std::ostream& bin_;
};
}  // namespace pass

namespace standin {
inline PartialShape parse_partial_shape(const std::string& text) {
    std::vector<Dimension> dims;
    std::string body = text.substr(1, text.size() - 2);
    std::stringstream ss(body);
    std::string item;
    while (std::getline(ss, item, ',')) dims.push_back(item == "?" ? Dimension::dynamic() : Dimension(std::stoll(item)));
    return PartialShape(dims);
}

// Reads what pass::Serialize wrote.
class Core : public ICore {
public:
    std::shared_ptr<Model> read_model(const std::string& text, const Tensor&, bool = false) const override {
        std::istringstream in(text);
        std::string line, magic, name;
        int version = 0;
        std::getline(in, line);
        {
            std::istringstream head(line);
            head >> magic >> version;
            std::getline(head, name);
            if (!name.empty() && name[0] == ' ') name.erase(0, 1);
        }
        OPENVINO_ASSERT(magic == "standin-ir" && version == 1, "not a stand-in model stream");
        std::vector<std::shared_ptr<Node>> nodes;
        ParameterVector params;
        ResultVector results;
        SinkVector sinks;
        std::map<std::string, std::shared_ptr<op::util::Variable>> variables;
        while (std::getline(in, line)) {
            if (line.empty()) continue;
            std::istringstream ls(line);
            size_t idx;
            std::string type, fname, inputs_kv, rest;
            ls >> idx >> type >> fname >> inputs_kv;
            std::getline(ls, rest);
            OutputVector inputs;
            {
                std::stringstream is(inputs_kv.substr(std::strlen("inputs=")));
                std::string item;
                while (std::getline(is, item, ',')) {
                    const size_t colon = item.find(':');
                    inputs.emplace_back(nodes.at(std::stoul(item.substr(0, colon))), std::stoul(item.substr(colon + 1)));
                }
            }
            std::map<std::string, std::string> attrs;
            {
                const size_t a = rest.find('{'), b = rest.rfind('}');
                std::stringstream as(rest.substr(a + 1, b - a - 1));
                std::string item;
                while (std::getline(as, item, ';')) {
                    const size_t eq = item.find('=');
                    if (eq != std::string::npos) attrs[item.substr(0, eq)] = item.substr(eq + 1);
                }
            }
            auto variable = [&]() {
                auto& v = variables[attrs.at("variable_id")];
                if (!v)
                    v = std::make_shared<op::util::Variable>(op::util::VariableInfo{
                        parse_partial_shape(attrs.at("variable_shape")), element::type_from_name(attrs.at("variable_type")),
                        attrs.at("variable_id")});
                return v;
            };
            std::shared_ptr<Node> n;
            if (type == "Parameter") {
                auto p = std::make_shared<op::v0::Parameter>(element::type_from_name(attrs.at("element_type")),
                                                             parse_partial_shape(attrs.at("shape")));
                params.push_back(p);
                n = p;
            } else if (type == "Result") {
                auto r = std::make_shared<op::v0::Result>(inputs.at(0));
                results.push_back(r);
                n = r;
            } else if (type == "Constant") {
                const std::string& hex = attrs.at("data");
                std::vector<uint8_t> bytes(hex.size() / 2);
                for (size_t i = 0; i < bytes.size(); i++) bytes[i] = (uint8_t)std::stoul(hex.substr(2 * i, 2), nullptr, 16);
                n = std::make_shared<op::v0::Constant>(element::type_from_name(attrs.at("element_type")),
                                                       parse_partial_shape(attrs.at("shape")).to_shape(), bytes.data());
            } else if (type == "ScaledDotProductAttention") {
                n = std::make_shared<op::v13::ScaledDotProductAttention>(inputs, attrs.at("causal") == "true");
            } else if (type == "PagedAttentionExtension") {
                auto pa = std::make_shared<op::PagedAttentionExtension>(inputs);
                for (int o = 0; o < 2; o++)
                    if (attrs.count("out" + std::to_string(o) + "_type"))
                        pa->set_out_type(o, element::type_from_name(attrs["out" + std::to_string(o) + "_type"]));
                n = pa;
            } else if (type == "ReadValue") {
                n = inputs.empty() ? std::make_shared<op::v6::ReadValue>(variable())
                                   : std::make_shared<op::v6::ReadValue>(inputs.at(0), variable());
            } else if (type == "Assign") {
                auto a = std::make_shared<op::v6::Assign>(inputs.at(0), variable());
                sinks.push_back(a);
                n = a;
            } else if (type == "Add") {
                n = std::make_shared<op::v1::Add>(inputs.at(0), inputs.at(1));
            } else if (type == "Subtract") {
                n = std::make_shared<op::v1::Subtract>(inputs.at(0), inputs.at(1));
            } else if (type == "Divide") {
                n = std::make_shared<op::v1::Divide>(inputs.at(0), inputs.at(1));
            } else if (type == "Softmax") {
                if (attrs.count("opset") && attrs["opset"] == "1")
                    n = std::make_shared<op::v1::Softmax>(inputs.at(0), (size_t)std::stoull(attrs.at("axis")));
                else
                    n = std::make_shared<op::v8::Softmax>(inputs.at(0), std::stoll(attrs.at("axis")));
            } else if (type == "Swish") {
                n = std::make_shared<op::v4::Swish>(inputs);
            } else if (type == "Multiply") {
                n = std::make_shared<op::v1::Multiply>(inputs.at(0), inputs.at(1));
            } else if (type == "GLU") {
                n = std::make_shared<op::internal::GLU>(
                    inputs.at(0), std::stoll(attrs.at("axis")), std::stoll(attrs.at("split_lengths")),
                    (op::internal::GLU::GluType)std::stoi(attrs.at("glu_type")), (size_t)std::stoull(attrs.at("split_to_glu_idx")),
                    attrs.count("output_type") ? element::type_from_name(attrs["output_type"]) : element::dynamic);
            } else if (type == "Reshape") {
                n = std::make_shared<op::v1::Reshape>(inputs.at(0), inputs.at(1), attrs.count("special_zero") && attrs["special_zero"] == "true");
            } else if (type == "Transpose") {
                n = std::make_shared<op::v1::Transpose>(inputs.at(0), inputs.at(1));
            } else if (type == "Squeeze") {
                n = std::make_shared<op::v0::Squeeze>(inputs);
            } else if (type == "Unsqueeze") {
                n = std::make_shared<op::v0::Unsqueeze>(inputs.at(0), inputs.at(1));
            } else if (type == "Convert") {
                n = std::make_shared<op::v0::Convert>(inputs.at(0), element::type_from_name(attrs.at("destination_type")));
            } else if (type == "MatMul") {
                n = std::make_shared<op::v0::MatMul>(inputs.at(0), inputs.at(1), attrs["transpose_a"] == "true",
                                                     attrs["transpose_b"] == "true");
            } else if (type == "Concat") {
                n = std::make_shared<op::v0::Concat>(inputs, std::stoll(attrs.at("axis")));
            } else if (type == "Gather") {
                n = std::make_shared<op::v8::Gather>(inputs.at(0), inputs.at(1), inputs.at(2),
                                                     attrs.count("batch_dims") ? std::stoll(attrs["batch_dims"]) : 0);
            } else if (type == "RMS") {
                n = std::make_shared<op::internal::RMS>(inputs.at(0), inputs.at(1), std::stod(attrs.at("epsilon")),
                                                        attrs.count("output_type") ? element::type_from_name(attrs["output_type"])
                                                                                   : element::dynamic);
            } else if (type == "RoPE") {
                op::internal::RoPE::Config c;
                auto num = [&](const char* k, size_t dflt) { return attrs.count(k) ? (size_t)std::stoull(attrs[k]) : dflt; };
                auto flag = [&](const char* k) { return attrs.count(k) && attrs[k] == "true"; };
                c.slice_start = num("slice_start", 0), c.slice_stop = num("slice_stop", 0);
                c.input_trans0213 = flag("input_trans0213"), c.output_trans0213 = flag("output_trans0213");
                c.is_interleaved = flag("is_interleaved"), c.rotary_ndims = num("rotary_ndims", 0);
                c.is_chatglm = flag("is_chatglm"), c.support_2d_rope = flag("support_2d_rope");
                c.is_qwen = flag("is_qwen"), c.use_rope_cache = flag("use_rope_cache");
                c.head_cnt = num("head_cnt", 0), c.head_size = num("head_size", 0);
                c.gather_position_arg_id = (int)num("gather_position_arg_id", 0);
                n = std::make_shared<op::internal::RoPE>(inputs, c);
            } else {
                OPENVINO_THROW("stand-in model stream holds an operator of type '", type, "'");
            }
            n->set_friendly_name(fname);
            for (size_t o = 0; o < n->get_output_size(); o++) n->output_names(o).insert(o ? fname + "." + std::to_string(o) : fname);
            OPENVINO_ASSERT(idx == nodes.size(), "stand-in model stream out of order");
            nodes.push_back(n);
        }
        return std::make_shared<Model>(results, sinks, params, name);
    }
};
}  // namespace standin

// ------------------------------------------------------------------------------ plugin API
class ICompiledModel;
class IAsyncInferRequest;
class ISyncInferRequest;
using SupportedOpsMap = std::map<std::string, std::string>;

class IPlugin : public std::enable_shared_from_this<IPlugin> {
public:
    IPlugin() : core_(std::make_shared<standin::Core>()) {}
    virtual ~IPlugin() = default;
    void set_version(const Version& v) { version_ = v; }
    const Version& get_version() const { return version_; }
    void set_device_name(const std::string& n) { device_name_ = n; }
    const std::string& get_device_name() const { return device_name_; }
    std::shared_ptr<ICore> get_core() const { return core_; }
    void set_core(const std::shared_ptr<ICore>& core) { core_ = core; }

    virtual void set_property(const AnyMap& properties) = 0;
    virtual Any get_property(const std::string& name, const AnyMap& arguments) const = 0;
    virtual std::shared_ptr<ICompiledModel> compile_model(const std::shared_ptr<const Model>& model,
                                                          const AnyMap& properties) const = 0;
    virtual std::shared_ptr<ICompiledModel> compile_model(const std::shared_ptr<const Model>& model,
                                                          const AnyMap& properties,
                                                          const SoPtr<IRemoteContext>& context) const = 0;
    virtual std::shared_ptr<ICompiledModel> import_model(std::istream& model, const AnyMap& properties) const = 0;
    virtual std::shared_ptr<ICompiledModel> import_model(std::istream& model, const SoPtr<IRemoteContext>& context,
                                                         const AnyMap& properties) const = 0;
    virtual std::shared_ptr<ICompiledModel> import_model(const Tensor& model, const AnyMap& properties) const = 0;
    virtual std::shared_ptr<ICompiledModel> import_model(const Tensor& model, const SoPtr<IRemoteContext>& context,
                                                         const AnyMap& properties) const = 0;
    virtual SupportedOpsMap query_model(const std::shared_ptr<const Model>& model, const AnyMap& properties) const = 0;
    virtual SoPtr<IRemoteContext> create_context(const AnyMap& remote_properties) const = 0;
    virtual SoPtr<IRemoteContext> get_default_context(const AnyMap& remote_properties) const = 0;

private:
    Version version_{"", ""};
    std::string device_name_;
    std::shared_ptr<ICore> core_;
};

// names of the nodes `is_node_supported` accepts, after `transform` has had its way with a copy of the model
inline std::unordered_set<std::string> get_supported_nodes(
    const std::shared_ptr<const Model>& model, std::function<void(std::shared_ptr<Model>&)> transform,
    std::function<bool(const std::shared_ptr<Node>)> is_node_supported, float = 1.0f) {
    auto copy = model->clone();
    transform(copy);
    std::unordered_set<std::string> names;
    for (const auto& n : copy->get_ordered_ops())
        if (is_node_supported(n)) names.insert(n->get_friendly_name());
    return names;
}

class ICompiledModel : public std::enable_shared_from_this<ICompiledModel> {
public:
    ICompiledModel(const std::shared_ptr<const Model>& model, const std::shared_ptr<const IPlugin>& plugin,
                   const std::shared_ptr<threading::ITaskExecutor>& task_executor = std::make_shared<threading::ImmediateExecutor>(),
                   const std::shared_ptr<threading::ITaskExecutor>& callback_executor = std::make_shared<threading::ImmediateExecutor>())
        : plugin_(plugin), task_executor_(task_executor), callback_executor_(callback_executor) {
        if (model) {
            inputs_ = model->inputs();
            outputs_ = model->outputs();
        }
    }
    virtual ~ICompiledModel() = default;
    virtual const std::vector<Output<const Node>>& inputs() const { return inputs_; }
    virtual const std::vector<Output<const Node>>& outputs() const { return outputs_; }
    virtual std::shared_ptr<IAsyncInferRequest> create_infer_request() const;
    virtual void export_model(std::ostream& model) const = 0;
    virtual std::shared_ptr<const Model> get_runtime_model() const = 0;
    virtual void set_property(const AnyMap& properties) = 0;
    virtual Any get_property(const std::string& name) const = 0;

protected:
    virtual std::shared_ptr<ISyncInferRequest> create_sync_infer_request() const = 0;
    std::shared_ptr<IAsyncInferRequest> create_async_infer_request() const;
    const std::shared_ptr<const IPlugin>& get_plugin() const { return plugin_; }
    const std::shared_ptr<threading::ITaskExecutor> get_task_executor() const { return task_executor_; }
    const std::shared_ptr<threading::ITaskExecutor> get_callback_executor() const { return callback_executor_; }
    void set_task_executor(const std::shared_ptr<threading::ITaskExecutor>& e) { task_executor_ = e; }
    void set_callback_executor(const std::shared_ptr<threading::ITaskExecutor>& e) { callback_executor_ = e; }

private:
    std::vector<Output<const Node>> inputs_, outputs_;
    std::shared_ptr<const IPlugin> plugin_;
    std::shared_ptr<threading::ITaskExecutor> task_executor_, callback_executor_;
};

class IInferRequest {
public:
    virtual ~IInferRequest() = default;
    virtual void infer() = 0;
    virtual std::vector<ProfilingInfo> get_profiling_info() const = 0;
    virtual SoPtr<ITensor> get_tensor(const Output<const Node>& port) const = 0;
    virtual void set_tensor(const Output<const Node>& port, const SoPtr<ITensor>& tensor) = 0;
    virtual std::vector<SoPtr<ITensor>> get_tensors(const Output<const Node>& port) const = 0;
    virtual void set_tensors(const Output<const Node>& port, const std::vector<SoPtr<ITensor>>& tensors) = 0;
    virtual std::vector<SoPtr<IVariableState>> query_state() const = 0;
    virtual const std::shared_ptr<const ICompiledModel>& get_compiled_model() const = 0;
    virtual const std::vector<Output<const Node>>& get_inputs() const = 0;
    virtual const std::vector<Output<const Node>>& get_outputs() const = 0;
};

class ISyncInferRequest : public IInferRequest {
public:
    explicit ISyncInferRequest(const std::shared_ptr<const ICompiledModel>& compiled_model) : compiled_model_(compiled_model) {}
    SoPtr<ITensor> get_tensor(const Output<const Node>& port) const override {
        auto it = tensors_.find(key(port));
        OPENVINO_ASSERT(it != tensors_.end(), "Cannot find tensor for port ", port.get_node()->get_friendly_name());
        return it->second;
    }
    void set_tensor(const Output<const Node>& port, const SoPtr<ITensor>& tensor) override {
        OPENVINO_ASSERT(is_port(port), "Cannot find tensor for port ", port.get_node()->get_friendly_name());
        OPENVINO_ASSERT(tensor, "Failed to set tensor: the tensor is not initialized");
        OPENVINO_ASSERT(port.get_element_type().compatible(tensor->get_element_type()),
                        "The tensor element type is not corresponding with output element type (",
                        tensor->get_element_type(), " != ", port.get_element_type(), ")");
        OPENVINO_ASSERT(port.get_partial_shape().compatible(PartialShape(tensor->get_shape())),
                        "The tensor shape ", tensor->get_shape(), " is not compatible with the port's ",
                        port.get_partial_shape());
        tensors_[key(port)] = tensor;
    }
    std::vector<SoPtr<ITensor>> get_tensors(const Output<const Node>&) const override { return {}; }
    void set_tensors(const Output<const Node>& port, const std::vector<SoPtr<ITensor>>& tensors) override {
        if (tensors.size() == 1) return set_tensor(port, tensors[0]);
        set_tensors_impl(port, tensors);
    }
    const std::shared_ptr<const ICompiledModel>& get_compiled_model() const override { return compiled_model_; }
    const std::vector<Output<const Node>>& get_inputs() const override { return compiled_model_->inputs(); }
    const std::vector<Output<const Node>>& get_outputs() const override { return compiled_model_->outputs(); }

protected:
    void check_tensors() const {
        for (const auto& port : get_inputs())
            OPENVINO_ASSERT(tensors_.count(key(port)), "input '", port.get_node()->get_friendly_name(), "' has not been set");
    }
    virtual void set_tensors_impl(const Output<const Node> port, const std::vector<SoPtr<ITensor>>& tensors) {
        (void)port;
        (void)tensors;
        OPENVINO_THROW_NOT_IMPLEMENTED("set_input_tensors/set_tensors are not supported by this plugin");
    }
    void allocate_tensor(const Output<const Node>& port, const std::function<void(SoPtr<ITensor>& tensor)>& allocate_callback) {
        allocate_callback(tensors_[key(port)]);
    }
    bool has_tensor(const Output<const Node>& port) const { return tensors_.count(key(port)) != 0; }

private:
    using Key = std::pair<const Node*, size_t>;
    static Key key(const Output<const Node>& port) { return {port.get_node(), port.get_index()}; }
    bool is_port(const Output<const Node>& port) const {
        for (const auto& p : get_inputs())
            if (p == port) return true;
        for (const auto& p : get_outputs())
            if (p == port) return true;
        return false;
    }
    std::shared_ptr<const ICompiledModel> compiled_model_;
    std::map<Key, SoPtr<ITensor>> tensors_;
};

// The staged asynchronous request: m_pipeline is a list of (executor, task); start_async hands
// stage 0 to its executor, each stage hands the next one on, wait() blocks until the last stage
// or an exception; cancel() lets the remaining stages be skipped and makes wait() throw
// ov::Cancelled; stop_and_wait() (for destructors) cancels what has not started and waits.
class IAsyncInferRequest : public IInferRequest {
public:
    IAsyncInferRequest(const std::shared_ptr<IInferRequest>& request,
                       const std::shared_ptr<threading::ITaskExecutor>& task_executor,
                       const std::shared_ptr<threading::ITaskExecutor>& callback_executor)
        : sync_request_(request), request_executor_(task_executor), callback_executor_(callback_executor) {
        m_pipeline = {{request_executor_, [this] { sync_request_->infer(); }}};
        m_sync_pipeline = m_pipeline;
    }
    ~IAsyncInferRequest() override { stop_and_wait(); }

    virtual void start_async() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (state_ == State::busy) throw Busy("Infer Request is busy");
            if (state_ == State::stopped) throw Exception("Infer Request was stopped");
            state_ = State::busy;
            cancel_requested_ = false;
            error_ = nullptr;
            done_ = std::promise<void>();
            done_future_ = done_.get_future().share();
        }
        try {
            start_async_thread_unsafe();
        } catch (...) {
            finish(std::current_exception());
            throw;
        }
    }
    virtual void wait() {
        std::shared_future<void> f;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            f = done_future_;
        }
        if (f.valid()) f.get();  // rethrows what a stage threw, or ov::Cancelled
    }
    virtual bool wait_for(const std::chrono::milliseconds& timeout) {
        std::shared_future<void> f;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            f = done_future_;
        }
        if (!f.valid()) return true;
        if (f.wait_for(timeout) != std::future_status::ready) return false;
        f.get();
        return true;
    }
    virtual void cancel() {
        std::lock_guard<std::mutex> lock(mutex_);
        if (state_ == State::busy) cancel_requested_ = true;
    }
    virtual void set_callback(std::function<void(std::exception_ptr)> callback) {
        std::lock_guard<std::mutex> lock(mutex_);
        callback_ = std::move(callback);
    }
    void infer() override {
        start_async();
        wait();
    }
    std::vector<ProfilingInfo> get_profiling_info() const override {
        check_not_busy();
        return sync_request_->get_profiling_info();
    }
    SoPtr<ITensor> get_tensor(const Output<const Node>& port) const override {
        check_not_busy();
        return sync_request_->get_tensor(port);
    }
    void set_tensor(const Output<const Node>& port, const SoPtr<ITensor>& tensor) override {
        check_not_busy();
        sync_request_->set_tensor(port, tensor);
    }
    std::vector<SoPtr<ITensor>> get_tensors(const Output<const Node>& port) const override {
        check_not_busy();
        return sync_request_->get_tensors(port);
    }
    void set_tensors(const Output<const Node>& port, const std::vector<SoPtr<ITensor>>& tensors) override {
        check_not_busy();
        sync_request_->set_tensors(port, tensors);
    }
    std::vector<SoPtr<IVariableState>> query_state() const override {
        check_not_busy();
        return sync_request_->query_state();
    }
    const std::shared_ptr<const ICompiledModel>& get_compiled_model() const override {
        return sync_request_->get_compiled_model();
    }
    const std::vector<Output<const Node>>& get_inputs() const override { return sync_request_->get_inputs(); }
    const std::vector<Output<const Node>>& get_outputs() const override { return sync_request_->get_outputs(); }

protected:
    using Stage = std::pair<std::shared_ptr<threading::ITaskExecutor>, threading::Task>;
    using Pipeline = std::vector<Stage>;
    void check_state() const { check_not_busy(); }
    void stop_and_wait() {
        std::shared_future<void> f;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (state_ == State::stopped) return;
            if (state_ == State::busy) cancel_requested_ = true;
            f = done_future_;
            callback_ = nullptr;
        }
        if (f.valid()) f.wait();
        std::lock_guard<std::mutex> lock(mutex_);
        state_ = State::stopped;
    }
    virtual void infer_thread_unsafe() { start_async_thread_unsafe(); }
    virtual void start_async_thread_unsafe() { run_stage(0); }
    Pipeline m_pipeline;
    Pipeline m_sync_pipeline;

private:
    enum class State { idle, busy, stopped };
    void check_not_busy() const {
        std::lock_guard<std::mutex> lock(mutex_);
        if (state_ == State::busy) throw Busy("Infer Request is busy");
    }
    void run_stage(size_t i) {
        if (i >= m_pipeline.size()) return finish(nullptr);
        m_pipeline[i].first->run([this, i] {
            bool cancelled;
            {
                std::lock_guard<std::mutex> lock(mutex_);
                cancelled = cancel_requested_;
            }
            if (cancelled) return finish(std::make_exception_ptr(Cancelled("Infer Request was canceled")));
            try {
                m_pipeline[i].second();
            } catch (...) {
                return finish(std::current_exception());
            }
            run_stage(i + 1);
        });
    }
    void finish(std::exception_ptr error) {
        std::function<void(std::exception_ptr)> callback;
        std::promise<void> done;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (state_ != State::busy) return;
            state_ = State::idle;
            callback = callback_;
            done = std::move(done_);
        }
        if (callback) {
            try {
                callback(error);
            } catch (...) {
                if (!error) error = std::current_exception();
            }
        }
        if (error)
            done.set_exception(error);
        else
            done.set_value();
    }
    std::shared_ptr<IInferRequest> sync_request_;
    std::shared_ptr<threading::ITaskExecutor> request_executor_, callback_executor_;
    mutable std::mutex mutex_;
    State state_ = State::idle;
    bool cancel_requested_ = false;
    std::exception_ptr error_;
    std::promise<void> done_;
    std::shared_future<void> done_future_;
    std::function<void(std::exception_ptr)> callback_;
};

inline std::shared_ptr<IAsyncInferRequest> ICompiledModel::create_async_infer_request() const {
    return std::make_shared<IAsyncInferRequest>(create_sync_infer_request(), task_executor_, callback_executor_);
}
inline std::shared_ptr<IAsyncInferRequest> ICompiledModel::create_infer_request() const {
    return create_async_infer_request();
}

}  // namespace ov

#define OV_DEFINE_PLUGIN_CREATE_FUNCTION(PluginType, version)                                               \
    extern "C" OPENVINO_PLUGIN_API void create_plugin_engine(::std::shared_ptr<::ov::IPlugin>& plugin);     \
    void create_plugin_engine(::std::shared_ptr<::ov::IPlugin>& plugin) {                                   \
        plugin = ::std::make_shared<PluginType>();                                                          \
        plugin->set_version(version);                                                                       \
    }
