// Shared helpers for the gfx950 kernels: error reporting across the C ABI, launch-shape helpers,
// wavefront (64-lane) reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/neoml_hip.h"

namespace nh {

// Stores the message returned by nhGetLastError() for the calling thread.
void setLastError( const char* fmt, ... );

inline hipStream_t toStream( nhStream s ) { return reinterpret_cast<hipStream_t>( s ); }

constexpr int WaveSize = 64;

inline int ceilDiv( long long a, long long b ) { return static_cast<int>( ( a + b - 1 ) / b ); }

inline bool isAligned16( const void* p ) { return ( reinterpret_cast<uintptr_t>( p ) & 15 ) == 0; }

} // namespace nh

// Argument check: the reference asserts, the C ABI returns NH_ERR_ARGUMENT.
#define NH_REQUIRE( expr ) \
	do { if( !( expr ) ) { nh::setLastError( "%s: requirement failed: %s", __func__, #expr ); return NH_ERR_ARGUMENT; } } while( 0 )

#define NH_HIP( call ) \
	do { hipError_t nhErr_ = ( call ); if( nhErr_ != hipSuccess ) { \
		nh::setLastError( "%s: %s failed: %s", __func__, #call, hipGetErrorString( nhErr_ ) ); return NH_ERR_HIP; } } while( 0 )

// After a kernel launch: report launch-configuration errors (asynchronous faults surface at the next sync).
#define NH_LAUNCH_CHECK() NH_HIP( hipGetLastError() )

#ifdef __HIPCC__
namespace nh {

__device__ __forceinline__ float waveReduceSum( float v )
{
#pragma unroll
	for( int off = 32; off > 0; off >>= 1 ) {
		v += __shfl_xor( v, off, 64 );
	}
	return v;
}

__device__ __forceinline__ float waveReduceMax( float v )
{
#pragma unroll
	for( int off = 32; off > 0; off >>= 1 ) {
		v = fmaxf( v, __shfl_xor( v, off, 64 ) );
	}
	return v;
}

} // namespace nh
#endif
