// Name -> factory registry of operators, filled at static-initialisation time by
// REGISTER_OPERATOR (reference utils/operator_registry.h:26-68).  Lookup and registration are
// serialised by one mutex; the operators themselves are not thread-safe.
#ifndef CATCCOS_HOST_OPERATOR_REGISTRY_H
#define CATCCOS_HOST_OPERATOR_REGISTRY_H

#include <mutex>
#include <unordered_map>
#include <vector>

#include "catccos_operator.h"

class OperatorRegistry {
public:
    static OperatorRegistry &Instance()
    {
        static OperatorRegistry instance;
        return instance;
    }

    // false when the name is already taken (the first registration wins)
    bool RegisterOperator(const std::string &opType, OperatorCreator creator)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        return registry_.emplace(opType, std::move(creator)).second;
    }

    // nullptr when the name is unknown
    std::unique_ptr<CatccosOperator> CreateOperator(const std::string &opType)
    {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = registry_.find(opType);
        return it == registry_.end() ? nullptr : it->second();
    }

    std::vector<std::string> Names()
    {
        std::lock_guard<std::mutex> lock(mutex_);
        std::vector<std::string> names;
        for (auto &kv : registry_) names.push_back(kv.first);
        return names;
    }

private:
    std::unordered_map<std::string, OperatorCreator> registry_;
    std::mutex mutex_;
};

#define REGISTER_OPERATOR(opType, opClass)                                                             \
    namespace {                                                                                        \
    struct opClass##Registrar {                                                                        \
        opClass##Registrar()                                                                           \
        {                                                                                              \
            OperatorRegistry::Instance().RegisterOperator(                                             \
                opType, []() -> std::unique_ptr<CatccosOperator> { return std::make_unique<opClass>(); }); \
        }                                                                                              \
    };                                                                                                 \
    static opClass##Registrar opClass##RegistrarInstance;                                              \
    }

#endif  // CATCCOS_HOST_OPERATOR_REGISTRY_H
