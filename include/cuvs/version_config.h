/*
 * API level of the cuVS release whose entry points this library mirrors (the reference generates
 * this header from its VERSION file, 26.10.00: cpp/CMakeLists.txt:36); cuvsVersionGet reports the
 * same numbers (c/src/core/c_api.cpp:274-280).
 */
#ifndef CUVS_AMD_VERSION_CONFIG_H
#define CUVS_AMD_VERSION_CONFIG_H

#define CUVS_VERSION_MAJOR 26
#define CUVS_VERSION_MINOR 10
#define CUVS_VERSION_PATCH 0

#endif
