// The CLI flag grammar a ROCm backend understands, as an exit-free parser shared by the command
// line front end and the embedded (C ABI) launcher.  Grammar of the reference's
// src/common/options.cpp:406-708; the embedded variant refuses --help / --version like
// parseCliOptionsNoExit does (src/common/options.cpp:732-749).
#pragma once
#include <string>
#include "mi355_peak.h"

enum class ParseResult { Ok, Help, Version, Error };

// Not part of clpeak's grammar: the shapes of the workloads (reduced ones for quick runs, the
// reference's constant operands).
struct HostExtras {
  Mi355Peak::Workload shape;
};

ParseResult parseCliCore(int argc, char **argv, CliOptions &opts, HostExtras &extras, std::string &error);
// false + message on anything but Ok.
bool parseCliOptionsNoExit(int argc, char **argv, CliOptions &opts, HostExtras &extras, std::string &error);
void printUsage(std::ostream &os);
