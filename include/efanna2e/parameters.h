// efanna2e::Parameters -- the string-to-string parameter map that carries CLI
// options into the index, with the interface of the reference's class
// (include/efanna2e/parameters.h:15-57): Set<T> stores operator<< text, Get<T>
// parses it back and throws std::invalid_argument for an unknown name,
// std::runtime_error for text that does not convert.
#pragma once
#include <map>
#include <sstream>
#include <stdexcept>
#include <string>
#include <typeinfo>

namespace efanna2e {

class Parameters {
   public:
    template <typename T>
    void Set(const std::string& name, const T& value) {
        std::ostringstream os;
        os << value;
        values_[name] = os.str();
    }

    template <typename T>
    T Get(const std::string& name) const {
        const auto it = values_.find(name);
        if (it == values_.end()) throw std::invalid_argument("Invalid parameter name.");
        return Convert<T>(it->second);
    }

    template <typename T>
    T Get(const std::string& name, const T& fallback) const {
        const auto it = values_.find(name);
        return it == values_.end() ? fallback : Convert<T>(it->second);
    }

   private:
    std::map<std::string, std::string> values_;

    template <typename T>
    static T Convert(const std::string& text) {
        std::istringstream is(text);
        T value;
        if (!(is >> value) || !is.eof())
            throw std::runtime_error("Failed to convert value '" + text + "' to type: " + typeid(T).name());
        return value;
    }
};

template <>
inline std::string Parameters::Convert<std::string>(const std::string& text) {
    return text;
}

}  // namespace efanna2e
