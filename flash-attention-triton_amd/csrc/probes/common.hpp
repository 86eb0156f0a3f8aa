// Shared by the measurement probes: a background reader of the shader clock and board power the
// driver publishes in sysfs.  The probes justify design choices of the kernels next door with
// numbers from the machine; they are not part of libfa2_gfx950.so.
#pragma once

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <glob.h>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_runtime.h>

#define HIP_CHECK(x)                                                                          \
  do {                                                                                        \
    hipError_t e_ = (x);                                                                      \
    if (e_ != hipSuccess) {                                                                   \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_));      \
      exit(1);                                                                                \
    }                                                                                         \
  } while (0)

struct SysfsSampler {
  std::string sclk_path, power_path;
  std::atomic<bool> stop{false};
  std::vector<double> sclk, power;
  std::thread worker;

  static std::string first_match(const char *pattern) {
    glob_t g;
    std::string r;
    if (glob(pattern, 0, nullptr, &g) == 0 && g.gl_pathc > 0) r = g.gl_pathv[0];
    globfree(&g);
    return r;
  }
  SysfsSampler() {
    sclk_path = first_match("/sys/class/drm/card*/device/pp_dpm_sclk");
    power_path = first_match("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average");
    if (power_path.empty()) power_path = first_match("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input");
  }
  static double read_sclk(const std::string &path) {  // the level marked '*', in MHz
    FILE *f = fopen(path.c_str(), "r");
    if (!f) return -1;
    char line[128];
    double mhz = -1;
    while (fgets(line, sizeof(line), f))
      if (strchr(line, '*')) {
        const char *c = strchr(line, ':');
        if (c) mhz = atof(c + 1);
      }
    fclose(f);
    return mhz;
  }
  static double read_watts(const std::string &path) {  // microwatts in the file
    FILE *f = fopen(path.c_str(), "r");
    if (!f) return -1;
    double uw = -1;
    if (fscanf(f, "%lf", &uw) != 1) uw = -1;
    fclose(f);
    return uw < 0 ? -1 : uw * 1e-6;
  }
  void start() {
    stop = false;
    sclk.clear();
    power.clear();
    worker = std::thread([this] {
      while (!stop) {
        if (!sclk_path.empty()) { double v = read_sclk(sclk_path); if (v > 0) sclk.push_back(v); }
        if (!power_path.empty()) { double v = read_watts(power_path); if (v > 0) power.push_back(v); }
        std::this_thread::sleep_for(std::chrono::milliseconds(20));
      }
    });
  }
  void finish() {
    stop = true;
    worker.join();
  }
  static double mean(const std::vector<double> &v) {
    if (v.empty()) return -1;
    double s = 0;
    for (double x : v) s += x;
    return s / v.size();
  }
};
