// Name -> factory registry with static-initialiser registration, the mechanism
// of dragon/core/registry.h:23-115.
#pragma once

#include "core/common.h"

namespace dragon {

template <class KeyT, class ObjectT, class... Args>
class Registry {
 public:
  typedef std::function<ObjectT*(Args...)> Creator;

  ObjectT* Create(const KeyT& key, Args... args) {
    auto it = registry_.find(key);
    CHECK(it != registry_.end()) << "\nKey(" << key << ") has not been registered.";
    return it->second(args...);
  }

  bool Has(const KeyT& key) const { return registry_.count(key) != 0; }

  void Register(const KeyT& key, Creator creator) {
    CHECK(!Has(key)) << "\nKey(" << key << ") has already been registered.";
    registry_[key] = creator;
  }

  vector<KeyT> keys() const {
    vector<KeyT> out;
    for (const auto& kv : registry_) out.push_back(kv.first);
    return out;
  }

 private:
  std::map<KeyT, Creator> registry_;
};

template <class KeyT, class ObjectT, class... Args>
class Registerer {
 public:
  Registerer(const KeyT& key, Registry<KeyT, ObjectT, Args...>* registry,
             typename Registry<KeyT, ObjectT, Args...>::Creator creator) {
    registry->Register(key, creator);
  }

  template <class DerivedT>
  static ObjectT* DefaultCreator(Args... args) {
    return new DerivedT(args...);
  }
};

#define DECLARE_TYPED_REGISTRY(RegistryName, KeyT, ObjectT, ...)              \
  ::dragon::Registry<KeyT, ObjectT, ##__VA_ARGS__>* RegistryName();           \
  typedef ::dragon::Registerer<KeyT, ObjectT, ##__VA_ARGS__> Registerer##RegistryName;

#define DEFINE_TYPED_REGISTRY(RegistryName, KeyT, ObjectT, ...)               \
  ::dragon::Registry<KeyT, ObjectT, ##__VA_ARGS__>* RegistryName() {          \
    static ::dragon::Registry<KeyT, ObjectT, ##__VA_ARGS__>* registry =       \
        new ::dragon::Registry<KeyT, ObjectT, ##__VA_ARGS__>();               \
    return registry;                                                          \
  }

#define DECLARE_REGISTRY(RegistryName, ObjectT, ...) \
  DECLARE_TYPED_REGISTRY(RegistryName, std::string, ObjectT, ##__VA_ARGS__)
#define DEFINE_REGISTRY(RegistryName, ObjectT, ...) \
  DEFINE_TYPED_REGISTRY(RegistryName, std::string, ObjectT, ##__VA_ARGS__)

#define REGISTER_CLASS(RegistryName, key, ...)                                   \
  static Registerer##RegistryName g_##RegistryName##_##key(                      \
      #key, RegistryName(), Registerer##RegistryName::DefaultCreator<__VA_ARGS__>);

} // namespace dragon
