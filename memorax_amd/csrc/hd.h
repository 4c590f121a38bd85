// Which head dim (d_k = d_v) this compilation of the chunked and single-step kernels serves.  The
// sources are compiled twice, for 64 and for 32.  The entry points of the 64 build are the public
// ones; they hand d_k = d_v = 32 on to those of the 32 build, which carry a suffix (MRX_API) and
// stay hidden inside the library.  Helpers with external linkage live in an inline namespace per
// build (MRX_HD_NS), so that the two sets of objects link into one library.
#pragma once
#ifndef MRX_HD
#define MRX_HD 64
#endif
#define MRX_CAT_(a, b) a##b
#define MRX_CAT(a, b) MRX_CAT_(a, b)
#if MRX_HD == 64
#define MRX_API(name) name
#define MRX_EXPORT extern "C"
#else
#define MRX_API(name) MRX_CAT(name, _hd32)
#define MRX_EXPORT extern "C" __attribute__((visibility("hidden")))
#endif
#define MRX_HD_NS MRX_CAT(hd, MRX_HD)
