// THRUST_CDNA4_HD: functions callable from kernels when the translation unit is compiled by hipcc;
// plain host functions under a host compiler.
#pragma once
#if defined(__HIPCC__)
#define THRUST_CDNA4_HD __host__ __device__
#else
#define THRUST_CDNA4_HD
#endif
