// --name=value command-line flags with the behaviour of the reference's scanner
// (cc/cuda_d_npeff/src/util/flag_util.h:30-143): the first argv entry that starts
// with "--name=" wins, required flags are fatal when missing ("Missing flag: name"),
// values go through std::stoi / std::stol / std::stof, and verify_no_unread() is
// fatal ("Unrecognized flags.") when the number of distinct flags read differs
// from argc - 1.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <set>
#include <stdexcept>
#include <string>

namespace hostutil {

[[noreturn]] inline void fatal(const std::string& msg) {
  std::printf("%s\n", msg.c_str());
  std::fflush(stdout);
  std::exit(1);
}

class Flags {
 public:
  Flags(int argc, char** argv) : argc_(argc), argv_(argv) {}

  bool find(const std::string& name, std::string* value) const {
    const std::string prefix = "--" + name + "=";
    for (int i = 0; i < argc_; i++) {
      std::string arg(argv_[i]);
      if (arg.rfind(prefix, 0) == 0) {
        *value = arg.substr(prefix.size());
        return true;
      }
    }
    return false;
  }

  void read(const std::string& name, std::string* out, bool required = true) {
    std::string v;
    if (!lookup(name, required, &v)) return;
    *out = v;
  }
  void read(const std::string& name, int* out, bool required = true) {
    std::string v;
    if (!lookup(name, required, &v)) return;
    *out = parse<int>(name, v, [](const std::string& s) { return std::stoi(s); });
  }
  void read(const std::string& name, long* out, bool required = true) {
    std::string v;
    if (!lookup(name, required, &v)) return;
    *out = parse<long>(name, v, [](const std::string& s) { return std::stol(s); });
  }
  void read(const std::string& name, float* out, bool required = true) {
    std::string v;
    if (!lookup(name, required, &v)) return;
    *out = parse<float>(name, v, [](const std::string& s) { return std::stof(s); });
  }

  bool unread_present() const { return (int)read_.size() != argc_ - 1; }
  void verify_no_unread() const {
    if (unread_present()) fatal("Unrecognized flags.");
  }

 private:
  bool lookup(const std::string& name, bool required, std::string* v) {
    if (!find(name, v)) {
      if (required) fatal("Missing flag: " + name);
      return false;
    }
    read_.insert(name);
    return true;
  }
  template <class T, class F>
  static T parse(const std::string& name, const std::string& v, F f) {
    try {
      return f(v);
    } catch (const std::exception&) {
      fatal("Invalid value for flag " + name + ": " + v);
    }
  }

  int argc_;
  char** argv_;
  std::set<std::string> read_;
};

}  // namespace hostutil
