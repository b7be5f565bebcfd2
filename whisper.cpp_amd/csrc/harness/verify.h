// Per-node parity of the MI355X backend against ggml's CPU backend inside the graphs a host really builds.
#pragma once

#include <string>

#include "ggml-backend.h"

namespace verify {

// dlopen the plugin, wrap graph_compute of every backend it creates, register it.  NULL if there is no device.
ggml_backend_reg_t load_plugin_hooked(const std::string & path);
void set_threads(int n);
void set_enabled(bool on);
void set_tolerance(double nmse);
// prints one JSON line per op kind seen since the last report (plus the first offending nodes); returns the number of
// nodes over tolerance
int  report(const char * phase);

} // namespace verify
