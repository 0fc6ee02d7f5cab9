// Seeded random fills for the benchmark's host buffers.
//
// Same overload set as the reference (Rand.h:7-28).  The reference draws floats from MKL's
// Niederreiter quasi-random stream (Rand.cc:20,35-41), which exists only inside MKL; here every
// value is a pure function of (seed, stream, counter), so any party that knows the three numbers
// regenerates the same inputs without sharing state:
//     raw(seed, stream, i) = mix64( mix64(seed + GOLDEN*(stream+1)) + GOLDEN*(i+1) )
//     uniform in [0,1)     = (raw >> 40) * 2^-24
//     standard normal      = sqrt(-2 ln u1) * cos(2 pi u2),  u1 = ((raw(2i)>>40)+1) * 2^-24,
//                                                            u2 =  (raw(2i+1)>>40)  * 2^-24
// with mix64 the splitmix64 finaliser and GOLDEN = 0x9E3779B97F4A7C15.
#pragma once

#include <cstddef>
#include <cstdint>

#include "AlignedVec.h"

// Restart the global stream.  Fills consume consecutive counters of the current stream;
// randStream(s) switches to stream s and rewinds its counter.
void randSeed(std::uint64_t seed);
void randStream(std::uint64_t stream);
std::uint64_t randRaw(std::uint64_t seed, std::uint64_t stream, std::uint64_t counter);

// Uniform fills.  `duplicates` only matters for the integer overloads: false = sample without
// replacement from [low, high].
void randFill(aligned_vector<float>& vec, const float low, const float high);
void randFill(aligned_vector<double>& vec, const double low, const double high);
void randFill(aligned_vector<int>& vec, const int low, const int high, bool duplicates = true);
void randFill(aligned_vector<std::int64_t>& vec, const int low, const int high,
              bool duplicates = true);
void randFill(float* array, std::size_t len, const float low, const float high,
              bool duplicates = true);
void randFill(double* array, std::size_t len, const double low, const double high,
              bool duplicates = true);
void randFill(int* array, int len, const int low, const int high, bool duplicates = true);
void randFill(std::int64_t* array, int len, const int low, const int high, bool duplicates = true);

// Normal(mean, stddev) fill (Box-Muller on the same stream; two counters per value).  The
// benchmark configs draw the upstream gradient dY from N(0,1).
void randFillNormal(float* array, std::size_t len, const float mean, const float stddev);
