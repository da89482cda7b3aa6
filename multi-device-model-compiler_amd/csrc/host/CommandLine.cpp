#include "multi-device-model-compiler/Runtime/CommandLine.h"

#include <cstdio>
#include <cstdlib>

namespace multi_device {
namespace cl {

namespace {
std::vector<Option *> &registry() {
  static std::vector<Option *> options;
  return options;
}

void splitCommas(const std::string &text, std::vector<std::string> &out) {
  size_t start = 0;
  while (true) {
    const size_t pos = text.find(',', start);
    out.emplace_back(text.substr(start, pos == std::string::npos ? pos : pos - start));
    if (pos == std::string::npos)
      break;
    start = pos + 1;
  }
}

void printHelp(const char *overview) {
  std::printf("OVERVIEW: %s\nOPTIONS:\n", overview);
  for (Option *o : registry()) {
    if (o->kind == Option::Positional)
      std::printf("  %-18s %s\n", "<positional>", o->desc.c_str());
    else
      std::printf("  --%-16s %s\n", o->name.c_str(), o->desc.c_str());
  }
}
} // namespace

Option::Option(Kind kind, const char *name, const char *desc, const char *init)
    : kind(kind), name(name), desc(desc), value(init) {
  initial_ = init;
  registry().push_back(this);
}

int Option::asInt() const { return std::atoi(value.c_str()); }
bool Option::asBool() const { return value == "1" || value == "true"; }

void ResetAllOptions() {
  for (Option *o : registry()) {
    o->value = o->initial_;
    o->values.clear();
    o->seen = false;
  }
}

bool ParseCommandLineOptions(int argc, char **argv, const char *overview) {
  for (int i = 1; i < argc; ++i) {
    std::string arg = argv[i];
    if (arg == "--help" || arg == "-help" || arg == "-h") {
      printHelp(overview);
      std::exit(0);
    }
    if (arg.size() > 1 && arg[0] == '-') {
      const size_t dashes = arg[1] == '-' ? 2 : 1;
      std::string name = arg.substr(dashes), value;
      bool hasValue = false;
      const size_t eq = name.find('=');
      if (eq != std::string::npos) {
        value = name.substr(eq + 1);
        name = name.substr(0, eq);
        hasValue = true;
      }
      Option *match = nullptr;
      for (Option *o : registry())
        if (o->kind != Option::Positional && o->name == name)
          match = o;
      if (!match) {
        std::fprintf(stderr, "%s: Unknown command line argument '%s'.  Try: '%s --help'\n", argv[0],
                     arg.c_str(), argv[0]);
        return false;
      }
      if (match->kind == Option::Bool) {
        match->value = hasValue ? value : "true";
      } else {
        if (!hasValue) {
          if (i + 1 >= argc) {
            std::fprintf(stderr, "%s: for the --%s option: requires a value!\n", argv[0],
                         name.c_str());
            return false;
          }
          value = argv[++i];
        }
        if (match->kind == Option::List)
          splitCommas(value, match->values);
        else
          match->value = value;
      }
      match->seen = true;
      continue;
    }
    Option *positional = nullptr;
    for (Option *o : registry())
      if (o->kind == Option::Positional && !o->seen) {
        positional = o;
        break;
      }
    if (!positional) {
      std::fprintf(stderr, "%s: Too many positional arguments specified!\n", argv[0]);
      return false;
    }
    positional->value = arg;
    positional->seen = true;
  }
  for (Option *o : registry())
    if (o->kind == Option::Positional && !o->seen) {
      std::fprintf(stderr, "%s: Not enough positional command line arguments specified!\nMust specify at least 1 positional argument: See: %s --help\n",
                   argv[0], argv[0]);
      return false;
    }
  return true;
}

} // namespace cl
} // namespace multi_device
