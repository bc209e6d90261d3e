// Stand-in for <gflags/gflags.h> (not installed here): the two macros fw_shim.cpp uses, with gflags' own meaning
// (DECLARE_x(name) declares the variable FLAGS_name that a DEFINE_x in another file defines).
#pragma once
#define DECLARE_bool(name) extern bool FLAGS_##name
#define DECLARE_double(name) extern double FLAGS_##name
