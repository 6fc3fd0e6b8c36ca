// String-keyed factories filled in by static initialisers, with the macro
// surface of shadow/core/registry.hpp:61-105 (SHADOW_DECLARE_REGISTRY,
// SHADOW_DEFINE_REGISTRY, SHADOW_REGISTER_CLASS).  Registering a key twice is a
// programming error and ends the process, as in shadow/core/registry.hpp:24-27.
// Registries are written during static initialisation only and read afterwards,
// so there is no locking.
#ifndef SHADOW_AMD_HOST_REGISTRY_HPP_
#define SHADOW_AMD_HOST_REGISTRY_HPP_

#include <cstdlib>
#include <functional>
#include <iostream>
#include <map>
#include <string>
#include <vector>

namespace Shadow {

template <typename Key, typename Object, typename... Args>
class Registry {
 public:
  using Creator = std::function<Object*(Args...)>;

  Registry() = default;
  Registry(const Registry&) = delete;
  Registry& operator=(const Registry&) = delete;

  void Register(const Key& key, Creator creator, const std::string& help = "") {
    if (!creators_.emplace(key, Entry{std::move(creator), help}).second) {
      std::cerr << "Key: " << key << " is already registered" << std::endl;
      std::exit(1);
    }
  }

  bool Has(const Key& key) const { return creators_.find(key) != creators_.end(); }

  // nullptr when the key is unknown; callers turn that into their own error.
  Object* Create(const Key& key, Args... args) const {
    auto it = creators_.find(key);
    return it == creators_.end() ? nullptr : it->second.make(args...);
  }

  std::vector<Key> Keys() const {
    std::vector<Key> keys;
    keys.reserve(creators_.size());
    for (const auto& kv : creators_) keys.push_back(kv.first);
    return keys;
  }

  std::string HelpMessage(const Key& key) const {
    auto it = creators_.find(key);
    return it == creators_.end() ? std::string() : it->second.help;
  }

 private:
  struct Entry {
    Creator make;
    std::string help;
  };
  std::map<Key, Entry> creators_;
};

// One of these per registration; its constructor does the work.
template <typename Key, typename Object, typename... Args>
struct Register {
  Register(const Key& key, Registry<Key, Object, Args...>* registry,
           typename Registry<Key, Object, Args...>::Creator creator, const std::string& help = "") {
    registry->Register(key, std::move(creator), help);
  }
  template <typename Derived>
  static Object* DefaultCreator(Args... args) {
    return new Derived(args...);
  }
};

}  // namespace Shadow

#define SHADOW_REGISTRY_CAT_(a, b) a##b
#define SHADOW_REGISTRY_CAT(a, b) SHADOW_REGISTRY_CAT_(a, b)

#define SHADOW_DECLARE_TYPED_REGISTRY(RegistryName, Key, Object, ...)  \
  ::Shadow::Registry<Key, Object, ##__VA_ARGS__>* RegistryName();      \
  using Register##RegistryName = ::Shadow::Register<Key, Object, ##__VA_ARGS__>;

// Function-local static: safe to use from other static initialisers.
#define SHADOW_DEFINE_TYPED_REGISTRY(RegistryName, Key, Object, ...)   \
  ::Shadow::Registry<Key, Object, ##__VA_ARGS__>* RegistryName() {     \
    static ::Shadow::Registry<Key, Object, ##__VA_ARGS__> instance;    \
    return &instance;                                                  \
  }

#define SHADOW_REGISTER_TYPED_CLASS(RegistryName, key, ...)                             \
  namespace {                                                                           \
  static Register##RegistryName SHADOW_REGISTRY_CAT(shadow_registered_, __COUNTER__)(  \
      key, RegistryName(), Register##RegistryName::DefaultCreator<__VA_ARGS__>);        \
  }

#define SHADOW_DECLARE_REGISTRY(RegistryName, Object, ...) \
  SHADOW_DECLARE_TYPED_REGISTRY(RegistryName, std::string, Object, ##__VA_ARGS__)
#define SHADOW_DEFINE_REGISTRY(RegistryName, Object, ...) \
  SHADOW_DEFINE_TYPED_REGISTRY(RegistryName, std::string, Object, ##__VA_ARGS__)
// The key is stringised: REGISTER(..., UnaryGPU(Default), ...) -> "UnaryGPU(Default)".
#define SHADOW_REGISTER_CLASS(RegistryName, key, ...) \
  SHADOW_REGISTER_TYPED_CLASS(RegistryName, #key, __VA_ARGS__)

#endif  // SHADOW_AMD_HOST_REGISTRY_HPP_
