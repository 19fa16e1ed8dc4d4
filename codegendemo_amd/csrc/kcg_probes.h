// kcg_probes.h — entry points of the GPU micro-benchmarks in kcg_probes.hip (see there).
#pragma once
int kcg_probe_mfma_peak(const char* dtype);   // "f16" (default) or "bf16"; prints one JSON line, returns 0
int kcg_probe_launch_cost();                  // prints two JSON lines, returns 0
