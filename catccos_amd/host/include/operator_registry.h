// Name -> factory registry of the operators (reference: utils/operator_registry.h:27-69).
#ifndef OPERATOR_REGISTRY_H
#define OPERATOR_REGISTRY_H

#include <mutex>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "catccos_operator.h"

class OperatorRegistry {
public:
    static OperatorRegistry& Instance()
    {
        static OperatorRegistry registry;      // constructed on first use, safe during static init
        return registry;
    }

    // true when the name was new; an existing registration is kept
    bool RegisterOperator(const std::string& op_type, OperatorCreator creator)
    {
        std::lock_guard<std::mutex> guard(mutex_);
        return creators_.emplace(op_type, std::move(creator)).second;
    }

    // a fresh operator object, or nullptr for an unknown name
    std::unique_ptr<CatccosOperator> CreateOperator(const std::string& op_type)
    {
        OperatorCreator creator;
        {
            std::lock_guard<std::mutex> guard(mutex_);
            const auto found = creators_.find(op_type);
            if (found == creators_.end()) {
                return nullptr;
            }
            creator = found->second;
        }
        return creator();
    }

    std::vector<std::string> RegisteredNames()
    {
        std::lock_guard<std::mutex> guard(mutex_);
        std::vector<std::string> names;
        for (const auto& kv : creators_) {
            names.push_back(kv.first);
        }
        return names;
    }

private:
    OperatorRegistry() = default;
    std::unordered_map<std::string, OperatorCreator> creators_;
    std::mutex mutex_;
};

// Registers op_class under op_type during static initialisation of the including translation unit.
#define REGISTER_OPERATOR(op_type, op_class)                                                              \
    class op_class;                                                                                       \
    namespace {                                                                                           \
    struct op_class##_registrar {                                                                         \
        op_class##_registrar()                                                                            \
        {                                                                                                 \
            OperatorRegistry::Instance().RegisterOperator(                                                \
                op_type, []() -> std::unique_ptr<CatccosOperator> { return std::make_unique<op_class>(); }); \
        }                                                                                                 \
    };                                                                                                    \
    static op_class##_registrar op_class##_instance;                                                      \
    }

#endif  // OPERATOR_REGISTRY_H
