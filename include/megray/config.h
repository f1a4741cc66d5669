// Build configuration of the MI355X virtual-rank MegRay library.
// The reference generates this file with CMake (include/megray/config.h.in:15-22); here the
// configuration is fixed: one HIP backend, nothing else.
#pragma once

#define MEGRAY_WITH_HIP
#define MEGRAY_WITH_VRANK

#ifndef MEGRAY_LOG_LEVEL
#define MEGRAY_LOG_LEVEL 2
#endif
