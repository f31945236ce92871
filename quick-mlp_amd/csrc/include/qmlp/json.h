#pragma once
// A small self-contained JSON value with the subset of the interface the QuickMLP
// host code needs (at / contains / value / get<T> / is_* / iteration / dump / parse).
// Objects keep their keys sorted, numbers keep the integer/float distinction.

#include <cstdint>
#include <initializer_list>
#include <map>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

namespace qmlp {

class json
{
public:
    enum class type_t { null, boolean, integer, number, string, array, object };
    typedef std::vector<json> array_t;
    typedef std::map<std::string, json> object_t;

    class parse_error : public std::runtime_error
    {
    public:
        explicit parse_error(const std::string& m) : std::runtime_error(m) {}
    };
    class type_error : public std::runtime_error
    {
    public:
        explicit type_error(const std::string& m) : std::runtime_error(m) {}
    };
    class out_of_range : public std::runtime_error
    {
    public:
        explicit out_of_range(const std::string& m) : std::runtime_error(m) {}
    };

    json() : type_(type_t::null) {}
    json(std::nullptr_t) : type_(type_t::null) {}
    json(bool v) : type_(type_t::boolean), bool_(v) {}
    json(int v) : type_(type_t::integer), int_(v) {}
    json(long v) : type_(type_t::integer), int_(v) {}
    json(long long v) : type_(type_t::integer), int_(v) {}
    json(unsigned v) : type_(type_t::integer), int_(v) {}
    json(unsigned long v) : type_(type_t::integer), int_(static_cast<int64_t>(v)) {}
    json(float v) : type_(type_t::number), num_(v) {}
    json(double v) : type_(type_t::number), num_(v) {}
    json(const char* v) : type_(type_t::string), str_(v) {}
    json(const std::string& v) : type_(type_t::string), str_(v) {}
    json(const array_t& v) : type_(type_t::array), arr_(v) {}
    json(const object_t& v) : type_(type_t::object), obj_(v) {}
    template <typename T>
    json(const std::vector<T>& v) : type_(type_t::array)
    {
        for (const auto& e : v) arr_.emplace_back(e);
    }

    static json array() { json j; j.type_ = type_t::array; return j; }
    static json array(std::initializer_list<json> l) { json j; j.type_ = type_t::array; j.arr_ = l; return j; }
    static json object() { json j; j.type_ = type_t::object; return j; }
    static json object(std::initializer_list<std::pair<const std::string, json>> l)
    {
        json j;
        j.type_ = type_t::object;
        for (const auto& kv : l) j.obj_[kv.first] = kv.second;
        return j;
    }

    static json parse(const std::string& text);
    [[nodiscard]] std::string dump(int indent = -1) const;

    [[nodiscard]] type_t type() const { return type_; }
    [[nodiscard]] bool is_null() const { return type_ == type_t::null; }
    [[nodiscard]] bool is_boolean() const { return type_ == type_t::boolean; }
    [[nodiscard]] bool is_number() const { return type_ == type_t::integer || type_ == type_t::number; }
    [[nodiscard]] bool is_number_integer() const { return type_ == type_t::integer; }
    [[nodiscard]] bool is_string() const { return type_ == type_t::string; }
    [[nodiscard]] bool is_array() const { return type_ == type_t::array; }
    [[nodiscard]] bool is_object() const { return type_ == type_t::object; }
    [[nodiscard]] const char* type_name() const;

    [[nodiscard]] size_t size() const
    {
        if (type_ == type_t::array) return arr_.size();
        if (type_ == type_t::object) return obj_.size();
        return type_ == type_t::null ? 0 : 1;
    }
    [[nodiscard]] bool empty() const { return size() == 0; }

    [[nodiscard]] bool contains(const std::string& key) const
    {
        return type_ == type_t::object && obj_.count(key) > 0;
    }
    [[nodiscard]] const json& at(const std::string& key) const
    {
        if (type_ != type_t::object) throw type_error(std::string("cannot use at(\"") + key + "\") with " + type_name());
        auto it = obj_.find(key);
        if (it == obj_.end()) throw out_of_range("key '" + key + "' not found");
        return it->second;
    }
    [[nodiscard]] const json& at(size_t i) const
    {
        if (type_ != type_t::array) throw type_error(std::string("cannot use at(index) with ") + type_name());
        if (i >= arr_.size()) throw out_of_range("array index out of range");
        return arr_[i];
    }
    json& operator[](const std::string& key)
    {
        if (type_ == type_t::null) type_ = type_t::object;
        if (type_ != type_t::object) throw type_error(std::string("cannot use operator[] with ") + type_name());
        return obj_[key];
    }
    const json& operator[](size_t i) const { return at(i); }
    void push_back(const json& v)
    {
        if (type_ == type_t::null) type_ = type_t::array;
        if (type_ != type_t::array) throw type_error(std::string("cannot use push_back with ") + type_name());
        arr_.push_back(v);
    }

    // iteration over arrays (objects: use items())
    [[nodiscard]] array_t::const_iterator begin() const { requireArray(); return arr_.begin(); }
    [[nodiscard]] array_t::const_iterator end() const { requireArray(); return arr_.end(); }
    [[nodiscard]] const object_t& items() const
    {
        if (type_ != type_t::object) throw type_error(std::string("cannot iterate items of ") + type_name());
        return obj_;
    }

    template <typename T>
    [[nodiscard]] T get() const
    {
        return getImpl(static_cast<T*>(nullptr));
    }
    template <typename T>
    [[nodiscard]] T value(const std::string& key, const T& fallback) const
    {
        if (type_ != type_t::object) throw type_error(std::string("cannot use value() with ") + type_name());
        auto it = obj_.find(key);
        if (it == obj_.end()) return fallback;
        return it->second.get<T>();
    }
    // implicit conversion to string, as used for "const std::string id = cfg.at("id")"
    operator std::string() const { return get<std::string>(); }

    bool operator==(const json& o) const;
    bool operator!=(const json& o) const { return !(*this == o); }

private:
    type_t type_;
    bool bool_ = false;
    int64_t int_ = 0;
    double num_ = 0;
    std::string str_;
    array_t arr_;
    object_t obj_;

    void requireArray() const
    {
        if (type_ != type_t::array) throw type_error(std::string("cannot iterate over ") + type_name());
    }
    bool getImpl(bool*) const
    {
        if (type_ != type_t::boolean) throw type_error(std::string("type must be boolean, but is ") + type_name());
        return bool_;
    }
    std::string getImpl(std::string*) const
    {
        if (type_ != type_t::string) throw type_error(std::string("type must be string, but is ") + type_name());
        return str_;
    }
    template <typename T, typename = std::enable_if_t<std::is_arithmetic<T>::value && !std::is_same<T, bool>::value>>
    T getImpl(T*) const
    {
        if (type_ == type_t::integer) return static_cast<T>(int_);
        if (type_ == type_t::number) return static_cast<T>(num_);
        if (type_ == type_t::boolean) return static_cast<T>(bool_);
        throw type_error(std::string("type must be number, but is ") + type_name());
    }
    template <typename T>
    std::vector<T> getImpl(std::vector<T>*) const
    {
        if (type_ != type_t::array) throw type_error(std::string("type must be array, but is ") + type_name());
        std::vector<T> out;
        out.reserve(arr_.size());
        for (const auto& e : arr_) out.push_back(e.get<T>());
        return out;
    }
    json getImpl(json*) const { return *this; }

    void dumpImpl(std::string& out, int indent, int level) const;
};

} // namespace qmlp
