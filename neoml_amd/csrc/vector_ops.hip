// Element-wise vector kernels (IVectorMathEngine). All of them stream through HBM once: 128-bit loads and
// stores, four independent 128-bit accesses per thread in flight, one workgroup per 4096 elements so that even a
// mid-sized vector spreads over all 256 compute units. Pointers that are not 16-byte aligned (handles with an
// element offset) take the scalar variant of the same kernel.
//
// Scalars that the engine keeps in device memory (thresholds, multipliers) are read inside the kernel.
// Results may alias an input exactly (in-place layers): every element is read before it is written by the
// same thread, so no __restrict__ is put on the pointers.
#include "common.h"
#include <float.h>
#include <map>
#include <mutex>
#include <stddef.h>
#include <type_traits>
#include <utility>

namespace nh {

constexpr int EltThreads = 256;
constexpr int EltUnroll = 4;

template<typename T> struct CVec4;
template<> struct CVec4<float> { typedef float4 Type; };
template<> struct CVec4<int> { typedef int4 Type; };

// 128-bit access with the streaming hint: the line is marked for early replacement in the caches. Vectors far larger
// than the caches are read and written once; measured on MI355X, a copy of 617 MB goes from 5.7 to 6.3 TB/s with it.
template<typename V> __device__ __forceinline__ V loadStreaming( const V* p )
{
	typedef unsigned raw4 __attribute__( ( ext_vector_type( 4 ) ) );
	const raw4 r = __builtin_nontemporal_load( reinterpret_cast<const raw4*>( p ) );
	V v;
	__builtin_memcpy( &v, &r, sizeof( V ) );
	return v;
}
template<typename V> __device__ __forceinline__ void storeStreaming( V* p, const V& v )
{
	typedef unsigned raw4 __attribute__( ( ext_vector_type( 4 ) ) );
	raw4 r;
	__builtin_memcpy( &r, &v, sizeof( V ) );
	__builtin_nontemporal_store( r, reinterpret_cast<raw4*>( p ) );
}

// STREAM bit 0: streaming loads, bit 1: streaming stores ( vector path only )
template<int NIN, typename TIn, typename TOut, typename F, bool VEC, int STREAM = 0>
__global__ __launch_bounds__( EltThreads )
void eltwiseKernel( const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, F f )
{
	f.prepare();
	if( VEC ) {
		typedef typename CVec4<TIn>::Type VIn;
		typedef typename CVec4<TOut>::Type VOut;
		const int n4 = n >> 2;
		const int base = blockIdx.x * ( EltThreads * EltUnroll ) + threadIdx.x;
		VIn va[EltUnroll], vb[EltUnroll], vc[EltUnroll];
#pragma unroll
		for( int u = 0; u < EltUnroll; ++u ) {
			const int i = base + u * EltThreads;
			if( i < n4 ) {
				if( ( STREAM & 1 ) != 0 ) {
					if( NIN >= 1 ) va[u] = loadStreaming( reinterpret_cast<const VIn*>( a ) + i );
					if( NIN >= 2 ) vb[u] = loadStreaming( reinterpret_cast<const VIn*>( b ) + i );
					if( NIN >= 3 ) vc[u] = loadStreaming( reinterpret_cast<const VIn*>( c ) + i );
				} else {
					if( NIN >= 1 ) va[u] = reinterpret_cast<const VIn*>( a )[i];
					if( NIN >= 2 ) vb[u] = reinterpret_cast<const VIn*>( b )[i];
					if( NIN >= 3 ) vc[u] = reinterpret_cast<const VIn*>( c )[i];
				}
			}
		}
#pragma unroll
		for( int u = 0; u < EltUnroll; ++u ) {
			const int i = base + u * EltThreads;
			if( i < n4 ) {
				VOut r;
				r.x = f( va[u].x, vb[u].x, vc[u].x );
				r.y = f( va[u].y, vb[u].y, vc[u].y );
				r.z = f( va[u].z, vb[u].z, vc[u].z );
				r.w = f( va[u].w, vb[u].w, vc[u].w );
				if( ( STREAM & 2 ) != 0 ) {
					storeStreaming( reinterpret_cast<VOut*>( out ) + i, r );
				} else {
					reinterpret_cast<VOut*>( out )[i] = r;
				}
			}
		}
		// tail of up to 3 elements
		if( blockIdx.x == 0 && threadIdx.x < ( n & 3 ) ) {
			const int i = ( n4 << 2 ) + threadIdx.x;
			const TIn x = NIN >= 1 ? a[i] : TIn();
			const TIn y = NIN >= 2 ? b[i] : TIn();
			const TIn z = NIN >= 3 ? c[i] : TIn();
			out[i] = f( x, y, z );
		}
	} else {
		const int base = blockIdx.x * ( EltThreads * EltUnroll * 4 ) + threadIdx.x;
#pragma unroll 4
		for( int u = 0; u < EltUnroll * 4; ++u ) {
			const int i = base + u * EltThreads;
			if( i < n ) {
				const TIn x = NIN >= 1 ? a[i] : TIn();
				const TIn y = NIN >= 2 ? b[i] : TIn();
				const TIn z = NIN >= 3 ? c[i] : TIn();
				out[i] = f( x, y, z );
			}
		}
	}
}

// A stream may put small calls aside and run several of them with one launch ( "tiny chains", below the functors ).
// true: the call has been taken over, nothing is left to launch.
template<int NIN, typename TIn, typename TOut, typename F>
static bool deferEltwise( nhStream s, const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, const F& f, int spread = TS_None,
	int width = 0, CSpreadAlone spreadAlone = nullptr );

template<int NIN, typename TIn, typename TOut, typename F>
static int launchEltwisePlain( hipStream_t stream, const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, F f );

template<int NIN, typename TIn, typename TOut, typename F>
static int launchEltwise( nhStream s, const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, F f )
{
	if( n < 0 ) {
		setLastError( "vector size is negative" );
		return NH_ERR_ARGUMENT;
	}
	if( n == 0 ) {
		return NH_OK;
	}
	if( out == nullptr || ( NIN >= 1 && a == nullptr ) || ( NIN >= 2 && b == nullptr ) || ( NIN >= 3 && c == nullptr ) ) {
		setLastError( "null vector pointer" );
		return NH_ERR_ARGUMENT;
	}
	if( deferEltwise<NIN, TIn, TOut, F>( s, a, b, c, out, n, f ) ) {
		return NH_OK;
	}
	return launchEltwisePlain<NIN, TIn, TOut, F>( toStream( s ), a, b, c, out, n, f );
}

// the launch of one call on its own ( operands checked by the caller )
template<int NIN, typename TIn, typename TOut, typename F>
static int launchEltwisePlain( hipStream_t stream, const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, F f )
{
	const bool vec = isAligned16( out ) && ( NIN < 1 || isAligned16( a ) ) && ( NIN < 2 || isAligned16( b ) )
		&& ( NIN < 3 || isAligned16( c ) ) && n >= 4;
	const int perBlock = EltThreads * EltUnroll * 4;
	const int blocks = ceilDiv( n, perBlock );
	// Vectors that cannot stay in the 256 MB last-level cache next to their result are read with the streaming hint
	// ( 51 M floats: 5.7 -> 6.8 TB/s ), the largest ones are written with it too ( 154 M floats: 5.8 -> 6.1 TB/s; for the
	// mid-sized ones streaming stores cost what streaming loads gain ). Below that the hint only loses cache hits.
	constexpr int StreamLoadsFrom = 24 << 20, StreamStoresFrom = 100 << 20;
	if( vec && NIN >= 1 && n >= StreamStoresFrom ) {
		hipLaunchKernelGGL( ( eltwiseKernel<NIN, TIn, TOut, F, true, 3> ), dim3( blocks ), dim3( EltThreads ), 0, stream,
			a, b, c, out, n, f );
	} else if( vec && NIN >= 1 && n >= StreamLoadsFrom ) {
		hipLaunchKernelGGL( ( eltwiseKernel<NIN, TIn, TOut, F, true, 1> ), dim3( blocks ), dim3( EltThreads ), 0, stream,
			a, b, c, out, n, f );
	} else if( vec ) {
		hipLaunchKernelGGL( ( eltwiseKernel<NIN, TIn, TOut, F, true> ), dim3( blocks ), dim3( EltThreads ), 0, stream,
			a, b, c, out, n, f );
	} else {
		hipLaunchKernelGGL( ( eltwiseKernel<NIN, TIn, TOut, F, false> ), dim3( blocks ), dim3( EltThreads ), 0, stream,
			a, b, c, out, n, f );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

// exp with the reference's clamps (src/CPU/x86/CpuX86.h:55: below -87.33654474 -> 0, above 88 -> FLT_MAX)
__device__ __forceinline__ float expClamped( float x )
{
	if( x < -87.33654474f ) {
		return 0.f;
	}
	if( x > 88.f ) {
		return FLT_MAX;
	}
	return expf( x );
}

// ---- functors: operator()( a, b, c ) with unused operands ignored ---------------------------------------

struct CNoScalar { __device__ void prepare() {} };

template<typename T> struct CCopyOp : CNoScalar { __device__ T operator()( T a, T, T ) const { return a; } };
template<typename T> struct CFillOp : CNoScalar { T Value; __device__ T operator()( T, T, T ) const { return Value; } };
template<typename T> struct CFillFromOp {
	const T* Ptr; T Value;
	__device__ void prepare() { Value = *Ptr; }
	__device__ T operator()( T, T, T ) const { return Value; }
};
struct CFloatToIntOp : CNoScalar { __device__ int operator()( float a, float, float ) const { return static_cast<int>( a ); } };
struct CIntToFloatOp : CNoScalar { __device__ float operator()( int a, int, int ) const { return static_cast<float>( a ); } };

struct CReLUOp {
	const float* Ptr; float Threshold;
	__device__ void prepare() { Threshold = *Ptr; }
	// max( x, 0 ) written so that NaN becomes 0, as _mm_max_ps( x, 0 ) does
	// (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:320-337)
	__device__ float operator()( float a, float, float ) const
	{
		float r = a > 0.f ? a : 0.f;
		if( Threshold > 0.f ) {
			r = r < Threshold ? r : Threshold;
		}
		return r;
	}
};
// ReLU of a sum: an element-wise sum whose launch waited for the ReLU behind it ( see CPendingSum )
struct CAddReLUOp {
	const float* Ptr; float Threshold;
	__device__ void prepare() { Threshold = *Ptr; }
	__device__ float operator()( float a, float b, float ) const
	{
		const float sum = a + b;
		float r = sum > 0.f ? sum : 0.f;
		if( Threshold > 0.f ) {
			r = r < Threshold ? r : Threshold;
		}
		return r;
	}
};
struct CELUOp {
	const float* Ptr; float Alpha;
	__device__ void prepare() { Alpha = *Ptr; }
	__device__ float operator()( float a, float, float ) const { return a >= 0.f ? a : Alpha * ( expClamped( a ) - 1.f ); }
};
struct CLeakyReLUOp {
	const float* Ptr; float Alpha;
	__device__ void prepare() { Alpha = *Ptr; }
	__device__ float operator()( float a, float, float ) const { return a > 0.f ? a : Alpha * a; }
};
struct CHSwishOp : CNoScalar {
	__device__ float operator()( float a, float, float ) const
	{
		if( a <= -3.f ) return 0.f;
		if( a >= 3.f ) return a;
		return a * ( a + 3.f ) * ( 1.f / 6.f );
	}
};
struct CMaxOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return a > b ? a : b; } };
struct CMinOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return a < b ? a : b; } };
struct CAbsOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return fabsf( a ); } };
struct CHardTanhOp : CNoScalar {
	__device__ float operator()( float a, float, float ) const { return a < -1.f ? -1.f : ( a > 1.f ? 1.f : a ); }
};
struct CHardSigmoidOp {
	const float* SlopePtr; const float* BiasPtr; float Slope, Bias;
	__device__ void prepare() { Slope = *SlopePtr; Bias = *BiasPtr; }
	__device__ float operator()( float a, float, float ) const
	{
		const float v = a * Slope + Bias;
		return v < 0.f ? 0.f : ( v > 1.f ? 1.f : v );
	}
};
struct CNegOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return -a; } };
struct CExpOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return expClamped( a ); } };
struct CLogOp : CNoScalar {
	// log( clamp( x, FLT_MIN, FLT_MAX ) ) (src/CPU/x86/CpuX86MathEngineVectorMathMkl.cpp:55-77)
	__device__ float operator()( float a, float, float ) const
	{
		float x = a > FLT_MIN ? a : FLT_MIN; // NaN -> FLT_MIN as std::max( x, FLT_MIN ) gives
		x = x < FLT_MAX ? x : FLT_MAX;
		return logf( x );
	}
};
struct CErfOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return erff( a ); } };
template<typename T> struct CAddOp : CNoScalar { __device__ T operator()( T a, T b, T ) const { return a + b; } };
template<typename T> struct CSubOp : CNoScalar { __device__ T operator()( T a, T b, T ) const { return a - b; } };
template<typename T> struct CMulOp : CNoScalar { __device__ T operator()( T a, T b, T ) const { return a * b; } };
struct CDivOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return a / b; } };
struct CNegMulOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return -a * b; } };
// result += first * second, two roundings like the reference's mul + add
// ( the product rounded by itself, as the CPU engine's separate multiply and add do: the pragma keeps the compiler from
// contracting the two into a fused multiply-add )
struct CMulAddOp : CNoScalar {
	__device__ float operator()( float a, float b, float c ) const
	{
#pragma clang fp contract( off )
		const float product = a * b;
		return c + product;
	}
};
template<typename T> struct CAddValueOp {
	const T* Ptr; T Value;
	__device__ void prepare() { Value = *Ptr; }
	__device__ T operator()( T a, T, T ) const { return a + Value; }
};
template<typename T> struct CMulValueOp {
	const T* Ptr; T Value;
	__device__ void prepare() { Value = *Ptr; }
	__device__ T operator()( T a, T, T ) const { return a * Value; }
};
struct CNegMulValueOp {
	const float* Ptr; float Value;
	__device__ void prepare() { Value = *Ptr; }
	__device__ float operator()( float a, float, float ) const { return -a * Value; }
};
// first + mult * second with separate rounding of the product
// (src/CPU/x86/CpuX86MathEngineVectorMathMkl.cpp:79-121)
struct CMultiplyAndAddOp {
	const float* Ptr; float Mult;
	__device__ void prepare() { Mult = *Ptr; }
	__device__ float operator()( float a, float b, float ) const
	{
#pragma clang fp contract( off )
		const float product = b * Mult;
		return a + product;
	}
};
struct CMultiplyAndSubOp {
	const float* Ptr; float Mult;
	__device__ void prepare() { Mult = *Ptr; }
	__device__ float operator()( float a, float b, float ) const
	{
#pragma clang fp contract( off )
		const float product = b * Mult;
		return a - product;
	}
};
struct CSqrtOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return sqrtf( a ); } };
struct CInvOp : CNoScalar {
	// saturating reciprocal (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:1321-1366):
	// -FLT_MIN <= x < 0 -> -FLT_MAX; 0 <= x <= FLT_MIN -> FLT_MAX. The reference runs with denormals-are-zero,
	// so a denormal of either sign counts as +0; the exponent bits are tested so that the answer does not depend
	// on the denormal mode of the comparison instructions.
	__device__ float operator()( float a, float, float ) const
	{
		if( ( __float_as_uint( a ) & 0x7f800000u ) == 0u ) return FLT_MAX;
		if( a == FLT_MIN ) return FLT_MAX;
		if( a == -FLT_MIN ) return -FLT_MAX;
		return 1.f / a;
	}
};
struct CMinMaxOp {
	const float* MinPtr; const float* MaxPtr; float Min, Max;
	__device__ void prepare() { Min = *MinPtr; Max = *MaxPtr; }
	__device__ float operator()( float a, float, float ) const
	{
		const float lo = a > Min ? a : Min;
		return lo < Max ? lo : Max;
	}
};
struct CSigmoidOp : CNoScalar {
	// e / ( e + 1 ), e = clamped exp( x ) (src/CPU/x86/CpuX86MathEngineVectorMathPrivate.h:1200-1228)
	__device__ float operator()( float a, float, float ) const
	{
		const float e = expClamped( a );
		return e / ( e + 1.f );
	}
};
struct CTanhOp : CNoScalar {
	// -1 + 2 / ( 1 + exp( -2x ) ) (src/CPU/x86/CpuX86MathEngineVectorMathPrivate.h:1178-1187);
	// tanhf is used for small |x| where that form loses relative accuracy through cancellation
	__device__ float operator()( float a, float, float ) const { return tanhf( a ); }
};

// ---- derivatives of the activations (backward pass): result = f'( first ) * second, or, for the ...DiffOp forms,
// the same derivative expressed through the activation's OUTPUT given as first
struct CNegLogOp : CNoScalar {
	// -log( clamp( x, FLT_MIN, FLT_MAX ) ): VectorLog with the sign flipped (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:1692-1720)
	__device__ float operator()( float a, float, float ) const
	{
		float x = a > FLT_MIN ? a : FLT_MIN;
		x = x < FLT_MAX ? x : FLT_MAX;
		return -logf( x );
	}
};
struct CReLUDiffOp {
	// second where 0 < first ( < threshold when the threshold is positive ), else 0; the same expression serves the
	// input and the output form (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:339-395)
	const float* Ptr; float Threshold;
	__device__ void prepare() { Threshold = *Ptr; }
	__device__ float operator()( float a, float b, float ) const
	{
		const bool pass = a > 0.f && ( Threshold <= 0.f || a < Threshold );
		return pass ? b : 0.f;
	}
};
struct CELUDiffOp {
	// first = the input: second where exp( first ) >= 1, else second * exp( first ) * alpha
	// (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:232-273)
	const float* Ptr; float Alpha;
	__device__ void prepare() { Alpha = *Ptr; }
	__device__ float operator()( float a, float b, float ) const
	{
		const float e = expClamped( a );
		return e >= 1.f ? b : b * e * Alpha;
	}
};
struct CELUDiffOutOp {
	// first = the output: second where first >= 0, else second * ( first + alpha ) (:275-318)
	const float* Ptr; float Alpha;
	__device__ void prepare() { Alpha = *Ptr; }
	__device__ float operator()( float a, float b, float ) const { return a >= 0.f ? b : b * ( a + Alpha ); }
};
struct CLeakyReLUDiffOp {
	// second above 0, second * alpha below, 0 at 0 as the reference's vector lanes have it (:394-432); the output
	// form is the same test, alpha being positive
	const float* Ptr; float Alpha;
	__device__ void prepare() { Alpha = *Ptr; }
	__device__ float operator()( float a, float b, float ) const { return a > 0.f ? b : ( a < 0.f ? b * Alpha : 0.f ); }
};
struct CHardTanhDiffOp : CNoScalar {
	// second inside ( -1, 1 ), else 0 (:783-812); serves the output form as well
	__device__ float operator()( float a, float b, float ) const { return ( -1.f < a && a < 1.f ) ? b : 0.f; }
};
struct CHardSigmoidDiffOp {
	// first = the input: second * slope inside ( -bias / slope, ( 1 - bias ) / slope ), else 0 (:825-875)
	const float* SlopePtr; const float* BiasPtr; float Slope, Low, High;
	__device__ void prepare() { Slope = *SlopePtr; const float bias = *BiasPtr; Low = -bias / Slope; High = ( 1.f - bias ) / Slope; }
	__device__ float operator()( float a, float b, float ) const { return ( Low < a && a < High ) ? b * Slope : 0.f; }
};
struct CHardSigmoidDiffOutOp {
	// first = the output: second * slope inside ( 0, 1 ), else 0 (:877-920)
	const float* SlopePtr; float Slope;
	__device__ void prepare() { Slope = *SlopePtr; }
	__device__ float operator()( float a, float b, float ) const { return ( 0.f < a && a < 1.f ) ? b * Slope : 0.f; }
};
struct CAbsDiffOp : CNoScalar {
	// second above 0, -second otherwise (:550-580)
	__device__ float operator()( float a, float b, float ) const { return a > 0.f ? b : -b; }
};
struct CSubValueOp {
	// first - Value, or Value - first when Reverse (the scalar forms of VectorSub)
	float Value; int Reverse;
	__device__ void prepare() {}
	__device__ float operator()( float a, float, float ) const { return Reverse ? Value - a : a - Value; }
};
// The element-wise parts of the hinge, squared hinge and Huber losses and of the L1 regulariser
// (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:584-782, 924-975, 1598-1640)
struct CHingeOp : CNoScalar { __device__ float operator()( float a, float, float ) const { return fmaxf( 0.f, 1.f - a ); } };
struct CSquaredHingeOp : CNoScalar {
	__device__ float operator()( float a, float, float ) const
	{
		if( a < -1.f ) return -4.f * a;
		const float t = fmaxf( 0.f, 1.f - a );
		return t * t;
	}
};
struct CHuberOp : CNoScalar {
	__device__ float operator()( float a, float, float ) const { return a > 1.f ? a - 0.5f : ( a < -1.f ? -a - 0.5f : a * a / 2 ); }
};
struct CHuberDerivativeOp : CNoScalar {
	__device__ float operator()( float a, float, float ) const { return a > 1.f ? 1.f : ( a < -1.f ? -1.f : a ); }
};
struct CHingeDiffOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return a < 1.f ? -b : 0.f; } };
struct CSquaredHingeDiffOp : CNoScalar {
	__device__ float operator()( float a, float b, float ) const
	{
		if( a < -1.f ) return -4.f * b;
		return -2.f * fmaxf( 0.f, 1.f - a ) * b;
	}
};
struct CL1DiffAddOp {
	// first + mult * clamp( second, -threshold, threshold )
	const float* ThresholdPtr; const float* MultPtr; float Threshold, Mult;
	__device__ void prepare() { Threshold = *ThresholdPtr; Mult = *MultPtr; }
	__device__ float operator()( float a, float b, float ) const
	{
		const float x = b < -Threshold ? -Threshold : ( b > Threshold ? Threshold : b );
		return a + Mult * x;
	}
};
struct CHSwishDiffOp : CNoScalar {
	// 0 below -3, second above 3, second * ( first / 3 + 1/2 ) between (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:433-480)
	__device__ float operator()( float a, float b, float ) const
	{
		if( !( -3.f < a ) ) return 0.f;
		return a < 3.f ? b * ( a * ( 1.f / 3.f ) + 0.5f ) : b;
	}
};
struct CSigmoidDiffOp : CNoScalar {
	// second / ( 2 + e + 1 / e ), e = clamped exp( -first ) (src/CPU/x86/CpuX86MathEngineVectorMath.cpp:1377-1412)
	__device__ float operator()( float a, float b, float ) const
	{
		const float e = expClamped( -a );
		return b / ( 2.f + e + 1.f / e );
	}
};
struct CSigmoidDiffOutOp : CNoScalar { __device__ float operator()( float y, float b, float ) const { return y * ( 1.f - y ) * b; } };
struct CTanhDiffOp : CNoScalar {
	__device__ float operator()( float a, float b, float ) const { const float t = tanhf( a ); return b * ( 1.f - t * t ); }
};
struct CTanhDiffOutOp : CNoScalar { __device__ float operator()( float y, float b, float ) const { return ( 1.f - y * y ) * b; } };

// ---- tiny chains -----------------------------------------------------------------------------------------------------
// A layer that normalises every row of a matrix ( CObjectNormalizationLayer::runOnceImpl,
// NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:181-242 ) asks for runs of element-wise calls over one value per row:
// a few thousand floats each, a launch of some 4 us that moves a few tens of KB. On a stream that has asked for it
// ( nhStreamDeferSmallOps ) such calls are put aside, up to TinyChainMax of them, and run by ONE launch as soon as
// anything else is asked of the stream ( toStream ), in the order of the calls and with the very functors of the
// separate launches, so every value is the same bit for bit.
//
// Inside that launch thread t of the grid handles elements t, t + threads, ... of every call. A call whose operands are
// either untouched by the calls in front of it in the chain, or begin exactly where an operand of one of them begins
// ( then each element is read and written by the same thread, in program order ), needs nothing between it and the
// call in front. Any other overlap ( a shifted view, a scalar that a call in front has produced ) needs every thread
// to have finished the calls in front: the chain then runs in one workgroup with a barrier in front of such calls ( calls
// over more than TinyOpMaxCount elements do not join such a chain: it is launched, and they begin the next one ).
//
// The same queue serves the passes of a layer over a whole blob: a call over more than TinyWideMaxCount elements begins
// a chain that only calls of its own count join ( an activation's or a solver's passes over one blob, the passes of a
// normalisation over its matrix, whose vectors per row or column are "spread" operands ). Such a chain never has barriers;
// it runs four elements per thread with 128-bit accesses where the operands allow it ( quadChainKernel ), through a kernel
// of its own if it is one of a few known sequences ( launchKnownChain ), and a call that nothing joined goes out as the
// launch it always was. In every chain without barriers whose calls have one count, a result that a later call
// overwrites before anything reads it from memory is computed but not stored ( CTinyOp::Dead ).

constexpr int TinyChainMax = 8;
constexpr int TinyOpMaxCount = 16384; // in a chain that runs as one workgroup
constexpr int TinyWideMaxCount = 262144; // in a chain without barriers whose calls differ in count ( a filter and its free terms )
constexpr int TinyThreads = 1024;
constexpr int TinyFunctorBytes = 16;

struct CTinyOp {
	const float* In[3];
	float* Out;
	const float* Scalar; // the device scalar that the functor reads when it starts ( host-side bookkeeping )
	int Count;
	short Kind; // index into CTinyKinds
	short Barrier; // every thread must have finished the calls in front
	alignas( 8 ) unsigned char Functor[TinyFunctorBytes];
	// The second operand of a call over a matrix of rows of Width elements may be a vector spread over it: one value per row
	// ( TS_PerRow: In[1][i / Width], AddVectorToMatrixColumns, MultiplyDiagMatrixByMatrix ) or per column ( TS_PerColumn:
	// In[1][i % Width], AddVectorToMatrixRows, MultiplyMatrixByDiagMatrix ). Only calls over more than TinyWideMaxCount
	// elements come with one, so a chain with barriers never holds any.
	short Spread;
	// The result is not stored: a later call of the chain writes the same elements, and every call in between that reads
	// them has them in registers ( chains without barriers whose calls all have one count; set when the chain is launched ).
	// NeoML's blobs of gradients are cleared, copied into, copied out of and cleared again in one run of calls.
	short Dead;
	int Width;
};

struct CTinyChain {
	int Length;
	int Blocks;
	int Straight; // no call has to wait for another: the grid has a thread per element of the longest call ( 4: per four elements )
	int Reserved;
	CTinyOp Ops[TinyChainMax];
};

template<typename... T> struct CTypeList {};
// the functors a chain may hold ( float in, float out, no more than TinyFunctorBytes of state )
typedef CTypeList<CFillOp<float>, CFillFromOp<float>, CCopyOp<float>, CAddOp<float>, CSubOp<float>, CMulOp<float>, CDivOp, CNegOp, CAbsOp, CMaxOp, CMinOp, CSqrtOp, CInvOp,
	CAddValueOp<float>, CMulValueOp<float>, CNegMulValueOp, CMultiplyAndAddOp, CMultiplyAndSubOp, CMulAddOp, CNegMulOp,
	CReLUOp, CSigmoidOp, CTanhOp, CHSwishOp> CTinyKinds;

template<typename F, typename List> struct CKindOf;
template<typename F> struct CKindOf<F, CTypeList<>> { static constexpr int Value = -1; };
template<typename F, typename Head, typename... Tail> struct CKindOf<F, CTypeList<Head, Tail...>> {
	static constexpr int Rest = CKindOf<F, CTypeList<Tail...>>::Value;
	static constexpr int Value = std::is_same<F, Head>::value ? 0 : ( Rest < 0 ? -1 : Rest + 1 );
};

template<typename F> __device__ __forceinline__ void runTinyOp( const CTinyOp& op, int first, int step )
{
	static_assert( sizeof( F ) <= TinyFunctorBytes && std::is_trivially_copyable<F>::value, "functor does not fit a chain" );
	F f;
	__builtin_memcpy( &f, op.Functor, sizeof( F ) );
	f.prepare();
	const float* a = op.In[0];
	const float* b = op.In[1];
	const float* c = op.In[2];
	for( int i = first; i < op.Count; i += step ) {
		const float x = a != nullptr ? a[i] : 0.f;
		const float y = b != nullptr ? b[i] : 0.f;
		const float z = c != nullptr ? c[i] : 0.f;
		op.Out[i] = f( x, y, z );
	}
}

template<typename List> struct CTinyDispatch;
template<> struct CTinyDispatch<CTypeList<>> {
	static __device__ __forceinline__ void Run( int, const CTinyOp&, int, int ) {}
};
template<typename Head, typename... Tail> struct CTinyDispatch<CTypeList<Head, Tail...>> {
	static __device__ __forceinline__ void Run( int kind, const CTinyOp& op, int first, int step )
	{
		if( kind == 0 ) {
			runTinyOp<Head>( op, first, step );
		} else {
			CTinyDispatch<CTypeList<Tail...>>::Run( kind - 1, op, first, step );
		}
	}
};

// N elements of one call, the functor's device scalar already in hand ( the functors that have one are { pointer, value }:
// the value sits behind the pointer )
template<typename F, int N> __device__ __forceinline__ void applyTinyOp( const CTinyOp& op, float scalar, const float* x, const float* y,
	const float* z, float* r )
{
	F f;
	__builtin_memcpy( &f, op.Functor, sizeof( F ) );
	if( sizeof( F ) == 16 && op.Scalar != nullptr ) {
		__builtin_memcpy( reinterpret_cast<char*>( &f ) + 8, &scalar, sizeof( float ) );
	}
#pragma unroll
	for( int i = 0; i < N; ++i ) {
		r[i] = f( x[i], y[i], z[i] );
	}
}

// ( the kind is the same for the whole grid: a search by halves costs a wavefront five scalar branches per call )
template<int I, typename List> struct CTypeAt;
template<typename Head, typename... Tail> struct CTypeAt<0, CTypeList<Head, Tail...>> { typedef Head Type; };
template<int I, typename Head, typename... Tail> struct CTypeAt<I, CTypeList<Head, Tail...>> {
	typedef typename CTypeAt<I - 1, CTypeList<Tail...>>::Type Type;
};
template<typename List> struct CTypeCount;
template<typename... T> struct CTypeCount<CTypeList<T...>> { static constexpr int Value = static_cast<int>( sizeof...( T ) ); };

template<typename List, int Lo = 0, int Hi = CTypeCount<List>::Value> struct CTinyApply {
	template<int N> static __device__ __forceinline__ void Run( int kind, const CTinyOp& op, float scalar, const float* x, const float* y,
		const float* z, float* r )
	{
		if constexpr( Hi - Lo == 1 ) {
			applyTinyOp<typename CTypeAt<Lo, List>::Type, N>( op, scalar, x, y, z, r );
		} else {
			constexpr int Mid = ( Lo + Hi ) / 2;
			if( kind < Mid ) {
				CTinyApply<List, Lo, Mid>::template Run<N>( kind, op, scalar, x, y, z, r );
			} else {
				CTinyApply<List, Mid, Hi>::template Run<N>( kind, op, scalar, x, y, z, r );
			}
		}
	}
};

// A chain in which no call waits for another, and a grid with a thread per Q * V elements of the longest call: a thread
// owns elements [first + u * stride, first + u * stride + V), u < Q, of every call ( V = 4: every call has the same count,
// a multiple of four, and operands on 16-byte boundaries; Q of these 128-bit accesses are in flight per operand, as in
// eltwiseKernel ). The scalars ( written by none of the calls ) are fetched together in front, and a call that reads where
// the call in front of it wrote, or what the first call read, takes the value from the register it is still in: one round
// trip to memory for a run of calls that work in place, not one per call.
template<int V> __device__ __forceinline__ void loadTinyValues( const float* p, float* v )
{
	if( V == 4 ) {
		const float4 q = *reinterpret_cast<const float4*>( p );
		v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
	} else {
		v[0] = *p;
	}
}

template<int V, int Q> __device__ __forceinline__ void runStraightChain( const CTinyChain& chain, long long first, int stride )
{
	constexpr int N = V * Q;
	float scalars[TinyChainMax];
#pragma unroll
	for( int k = 0; k < TinyChainMax; ++k ) {
		scalars[k] = k < chain.Length && chain.Ops[k].Scalar != nullptr ? *chain.Ops[k].Scalar : 0.f;
	}
	const float* lastOut = nullptr; // what the call in front wrote
	float lastValue[N] = {};
	bool lastMine[Q] = {};
	const float* heldIn = nullptr; // what the first call read ( its first operand ), and what has been written there since
	float heldValue[N] = {};
	bool heldMine[Q] = {};
	int spreadWidth = 0; // where the thread's elements lie in a matrix of rows of that many elements
	unsigned row[Q] = {}, column[Q] = {};
#pragma unroll
	for( int k = 0; k < TinyChainMax; ++k ) {
		if( k >= chain.Length ) {
			break;
		}
		const CTinyOp& op = chain.Ops[k];
		bool mine[Q];
#pragma unroll
		for( int u = 0; u < Q; ++u ) {
			mine[u] = first + static_cast<long long>( u ) * stride < op.Count;
		}
		float in[3][N] = {};
#pragma unroll
		for( int j = 0; j < 3; ++j ) {
			if( op.In[j] == nullptr ) {
				continue;
			}
			if( j == 1 && op.Spread != TS_None ) {
				if( op.Width != spreadWidth ) {
					// ( the divisions once per width: the calls of a chain are as a rule over one matrix )
					spreadWidth = op.Width;
#pragma unroll
					for( int u = 0; u < Q; ++u ) {
						const unsigned element = static_cast<unsigned>( first + static_cast<long long>( u ) * stride );
						row[u] = element / static_cast<unsigned>( spreadWidth );
						column[u] = element - row[u] * static_cast<unsigned>( spreadWidth );
					}
				}
#pragma unroll
				for( int u = 0; u < Q; ++u ) {
					if( !mine[u] ) {
						continue;
					}
					// ( with V = 4 the width is a multiple of four: the four elements lie in one row, on four columns in a row )
					if( op.Spread == TS_PerRow ) {
						const float value = op.In[1][row[u]];
#pragma unroll
						for( int v = 0; v < V; ++v ) in[1][u * V + v] = value;
					} else {
						loadTinyValues<V>( op.In[1] + column[u], &in[1][u * V] );
					}
				}
				continue;
			}
			const bool fromLast = op.In[j] == lastOut, fromHeld = op.In[j] == heldIn;
#pragma unroll
			for( int u = 0; u < Q; ++u ) {
				if( !mine[u] ) {
					continue;
				}
				if( fromLast && lastMine[u] ) {
#pragma unroll
					for( int v = 0; v < V; ++v ) in[j][u * V + v] = lastValue[u * V + v];
				} else if( fromHeld && heldMine[u] ) {
#pragma unroll
					for( int v = 0; v < V; ++v ) in[j][u * V + v] = heldValue[u * V + v];
				} else {
					loadTinyValues<V>( op.In[j] + first + static_cast<long long>( u ) * stride, &in[j][u * V] );
				}
			}
		}
		if( k == 0 && op.In[0] != nullptr ) {
			heldIn = op.In[0];
#pragma unroll
			for( int u = 0; u < Q; ++u ) heldMine[u] = mine[u];
#pragma unroll
			for( int i = 0; i < N; ++i ) heldValue[i] = in[0][i];
		}
		// ( elements that are not the thread's are computed from zeros and go nowhere )
		CTinyApply<CTinyKinds>::template Run<N>( op.Kind, op, scalars[k], in[0], in[1], in[2], lastValue );
		const bool overHeld = op.Out == heldIn;
#pragma unroll
		for( int u = 0; u < Q; ++u ) {
			if( mine[u] && op.Dead == 0 ) {
				float* to = op.Out + first + static_cast<long long>( u ) * stride;
				if( V == 4 ) {
					*reinterpret_cast<float4*>( to ) = make_float4( lastValue[u * V], lastValue[u * V + 1], lastValue[u * V + 2], lastValue[u * V + 3] );
				} else {
					*to = lastValue[u * V];
				}
			}
			if( overHeld ) {
				// ( whoever writes there owns the same elements: the held value follows )
				heldMine[u] = mine[u];
#pragma unroll
				for( int v = 0; v < V; ++v ) heldValue[u * V + v] = lastValue[u * V + v];
			}
			lastMine[u] = mine[u];
		}
		lastOut = op.Out;
	}
}

__global__ __launch_bounds__( TinyThreads ) void tinyChainKernel( const CTinyChain chain )
{
	const int first = blockIdx.x * blockDim.x + threadIdx.x;
	const int step = gridDim.x * blockDim.x;
	if( chain.Straight != 0 ) {
		runStraightChain<1, 1>( chain, first, 0 );
		return;
	}
	for( int k = 0; k < chain.Length; ++k ) {
		const CTinyOp& op = chain.Ops[k];
		if( op.Barrier != 0 ) {
			// only in chains of one workgroup; the stores in front are visible to the whole workgroup behind it
			__syncthreads();
		}
		CTinyDispatch<CTinyKinds>::Run( op.Kind, op, first, step );
	}
}

// the same for calls of one count over vectors on 16-byte boundaries: QuadsPerThread times four elements per thread
// ( the three calls of a GELU over 16.7 M elements: 72.6 us as three launches, 69 us with one quad per thread, 50 us with four )
// ( the four last calls of a normalisation layer over 8192 x 512 values, 16 MB that stay in the caches: 25 us as four launches,
// 12 us as one, with one quad per thread as with four: what is left is a wavefront waiting for one call's spread vector
// after the other )
constexpr int QuadThreads = 256, QuadsPerThread = 4;
__global__ __launch_bounds__( QuadThreads ) void quadChainKernel( const CTinyChain chain )
{
	runStraightChain<4, QuadsPerThread>( chain,
		4ll * ( static_cast<long long>( blockIdx.x ) * ( QuadThreads * QuadsPerThread ) + threadIdx.x ), 4 * QuadThreads );
}

// A product A * B^T whose launch waits for the call behind it: a fully connected layer ( CFullyConnectedLayer::RunOnce,
// NeoML/src/Dnn/Layers/FullyConnectedLayer.cpp:91-99 ) asks for the product and then for its free term to be added to the
// product's rows in place, a pass over the whole result for one add per element. On a stream that puts small calls aside
// the product is put aside too ( nothing else is pending then ), and if the next call is that AddVectorToMatrixRows, both
// go out as the one launch the product's kernels have for it ( the free term added to the accumulators on their way
// out ); any other call launches the product as it was asked for, first.
struct CPendingProduct {
	bool Pending = false;
	const float* A = nullptr;
	const float* B = nullptr;
	float* C = nullptr;
	int Lda = 0, Ldb = 0, Ldc = 0, M = 0, N = 0, K = 0;
};

// A convolution ( plain or channelwise ) that waits for the call behind it in the same way: CConvLayer / CChannelwiseConvLayer
// are followed by CReLULayer in most networks, a pass over the whole result in place that the convolution's kernels do on
// the accumulators' way out ( nhBlobConvolutionWithActivation ). VectorReLU over the convolution's result in place makes
// the two one launch, the threshold read from where the engine keeps it in device memory.
struct CPendingConvolution {
	bool Pending = false;
	bool Channelwise = false;
	nhConvDesc Desc = {};
	const float* Source = nullptr;
	const float* Filter = nullptr;
	const float* FreeTerm = nullptr;
	float* Result = nullptr;
};

// The sum of two large vectors ( the junction of a residual block, CEltwiseSumLayer ) followed by CReLULayer in place:
// one pass instead of two.
struct CPendingSum {
	bool Pending = false;
	const float* First = nullptr;
	const float* Second = nullptr;
	float* Result = nullptr;
	int Count = 0;
};

// A batch of small products C[b] = A[b] * B[b] ( dense, row-major ) followed by VectorMultiply over the whole result in place
// by a device scalar: CMatrixMultiplicationLayer + CLinearLayer, the scores of an attention layer and their 1 / sqrt( d )
// ( NeoML/src/Dnn/Layers/MultiheadAttentionLayer.cpp:168-183 ). The kernel for such batches multiplies on the way out.
struct CPendingBatched {
	bool Pending = false;
	const float* A = nullptr;
	const float* B = nullptr;
	float* C = nullptr;
	int Batch = 0, M = 0, N = 0, K = 0;
};

// The sums of the rows of a matrix ( SumMatrixColumns: one value per row ) followed by element-wise calls with one operand
// in place over those sums: the mean and the inverse deviation of CObjectNormalizationLayer ( sum, x -1/width; sum, x 1/width,
// + epsilon, sqrt, 1/x ). The sum waits; such calls are queued behind it as its tail ( the queue's chain holds nothing else
// while it waits ), and the launch of the sum applies them to each row's value before it is stored, with the calls' own
// functors: one launch for the reduction and its tail. Any other call launches the sum with the tail it has by then.
struct CPendingColumnSum {
	bool Pending = false;
	float* Result = nullptr;
	const float* Matrix = nullptr;
	int Height = 0, Width = 0;
	// The matrix may itself be a sum of two that waited on the stream ( VectorAdd over the whole matrix: the residual sum in
	// front of a normalisation ): the launch then adds the two, writes the matrix and sums its rows in one pass.
	const float* AddFirst = nullptr;
	const float* AddSecond = nullptr;
	// ... or the squares of a matrix's distances from a value per row, the two calls in front of a normalisation's variance
	// that waited as a chain ( matrix = ( SquareOf + SquareShift[row] )^2 ): computed, written and summed in one pass.
	const float* SquareOf = nullptr;
	const float* SquareShift = nullptr;
};

struct CTinyQueue {
	bool Enabled = false;
	CTinyChain Chain = {};
	// A call over more than TinyWideMaxCount elements begins a chain that only calls of the same count join ( the passes
	// of an activation or of a solver over one blob, quadChainKernel ); if none does, the call goes out as the launch it
	// would have been on any other stream:
	void ( *FirstAlone )( hipStream_t, const CTinyOp& ) = nullptr;
	CSpreadAlone FirstSpreadAlone = nullptr; // ( the same for a call with a spread operand: its own kernel lives with its entry point )
	CPendingProduct Product;
	CPendingConvolution Convolution;
	CPendingSum Sum;
	CPendingBatched Batched;
	CPendingPadding Padding;
	CPendingColumnSum ColumnSum;

	bool LaunchWaits() const
	{
		return Product.Pending || Convolution.Pending || Sum.Pending || Batched.Pending || Padding.Pending || ColumnSum.Pending;
	}
};

static int launchPlainSum( hipStream_t stream, const CPendingSum& sum );

int launchDeferredConvolution( hipStream_t stream, bool channelwise, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result, const CFusedActivation& act );

int matMulNT( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC, const float* bias, bool accumulate );

int matMulNN( hipStream_t stream, const float* a, int lda, const float* b, int ldb, float* c, int ldc,
	int M, int N, int K, int batch, long long strideA, long long strideB, long long strideC, bool accumulate,
	const float* scale, bool* scaled );

static int launchBatched( hipStream_t stream, const CPendingBatched& p, const float* scale, bool* scaled )
{
	return matMulNN( stream, p.A, p.K, p.B, p.N, p.C, p.N, p.M, p.N, p.K, p.Batch, static_cast<long long>( p.M ) * p.K,
		static_cast<long long>( p.K ) * p.N, static_cast<long long>( p.M ) * p.N, false, scale, scaled );
}

typedef std::map<std::pair<int, hipStream_t>, CTinyQueue> CTinyQueues;
// ( recursive: a product launched from under the lock may ask its stream's pool for scratch memory, a pool at its limit
// gives memory back first, and giving memory back launches what every stream holds )
static std::recursive_mutex tinyLock;
static CTinyQueues& tinyQueues()
{
	static CTinyQueues* queues = new CTinyQueues; // never destroyed: calls may still arrive while the process unloads
	return *queues;
}
int tinyChainsPending = 0;
static int tinyDeferringStreams = 0;

// With tinyLock held and the queue's device current. true: something was launched ( telling a stream's one-launch LSTMs
// about it, noteStreamUse, is left to the callers: that takes a lock that a caller of toStream may hold ).
// ---- chains whose calls are known when the library is compiled ------------------------------------------------------------
// quadChainKernel finds out per call and wavefront what the call is and where each operand's values are, about 900 cycles
// that a chain over 8192 x 512 values feels ( 1.5 us per call ). Three sequences that NeoML's layers ask for at that size
// have a kernel of their own, with the very functors or expressions of the separate calls ( contraction into fused
// multiply-adds switched off where a product of one call meets a sum of the next ), so the bits stay those of the separate
// launches; anything else, and any other layout of the same calls, runs through quadChainKernel.
constexpr int KnownQuads = 4; // 128-bit accesses in flight per thread and operand

// CGELULayer::runFastApproximate ( NeoML/src/Dnn/Layers/GELULayer.cpp:145-160 ): t = x * scale; t = sigmoid( t ); out = x * t,
// out being t or another vector ( then t is written too )
__global__ __launch_bounds__( 256 ) void geluChainKernel( const float* x, float* t, float* out, const float* scale, int quads )
{
	CMulValueOp<float> byScale; byScale.Ptr = scale; byScale.prepare();
	const CSigmoidOp sigmoid;
	const CMulOp<float> product;
	const int base = blockIdx.x * ( 256 * KnownQuads ) + threadIdx.x;
	float4 in[KnownQuads];
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
			in[u] = reinterpret_cast<const float4*>( x )[i];
		}
	}
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
			const float v[4] = { in[u].x, in[u].y, in[u].z, in[u].w };
			float gate[4], result[4];
#pragma unroll
			for( int e = 0; e < 4; ++e ) {
				gate[e] = sigmoid( byScale( v[e], 0.f, 0.f ), 0.f, 0.f );
				result[e] = product( v[e], gate[e], 0.f );
			}
			if( out != t ) {
				reinterpret_cast<float4*>( t )[i] = make_float4( gate[0], gate[1], gate[2], gate[3] );
			}
			reinterpret_cast<float4*>( out )[i] = make_float4( result[0], result[1], result[2], result[3] );
		}
	}
}

// The four last calls of CObjectNormalizationLayer::runOnceImpl ( NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:213-242 ):
// y = x + negMean[row]; y *= invDeviation[row]; out = y * scale[column]; out += bias[column], out being y or another
// matrix ( then y is written too ). With squared: the two calls in front of the variance, y = x + negMean[row]; y *= y.
template<bool SQUARED>
__global__ __launch_bounds__( 256 ) void normalizeChainKernel( const float* x, float* y, float* out, const float* negMean,
	const float* invDeviation, const float* scale, const float* bias, int width, int quads )
{
	const int base = blockIdx.x * ( 256 * KnownQuads ) + threadIdx.x;
	float4 in[KnownQuads], byColumn[KnownQuads], toColumn[KnownQuads];
	float toRow[KnownQuads], byRow[KnownQuads];
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
			const unsigned element = static_cast<unsigned>( i ) * 4u;
			const unsigned row = element / static_cast<unsigned>( width );
			const unsigned column = element - row * static_cast<unsigned>( width );
			in[u] = reinterpret_cast<const float4*>( x )[i];
			toRow[u] = negMean[row];
			if( !SQUARED ) {
				byRow[u] = invDeviation[row];
				byColumn[u] = *reinterpret_cast<const float4*>( scale + column );
				toColumn[u] = *reinterpret_cast<const float4*>( bias + column );
			}
		}
	}
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
#pragma clang fp contract( off )
			const float v[4] = { in[u].x, in[u].y, in[u].z, in[u].w };
			float centred[4], result[4];
			if( SQUARED ) {
#pragma unroll
				for( int e = 0; e < 4; ++e ) {
					centred[e] = v[e] + toRow[u];
					result[e] = centred[e] * centred[e];
				}
			} else {
				const float s[4] = { byColumn[u].x, byColumn[u].y, byColumn[u].z, byColumn[u].w };
				const float b[4] = { toColumn[u].x, toColumn[u].y, toColumn[u].z, toColumn[u].w };
#pragma unroll
				for( int e = 0; e < 4; ++e ) {
					centred[e] = v[e] + toRow[u];
					centred[e] = centred[e] * byRow[u];
					result[e] = centred[e] * s[e];
					result[e] = result[e] + b[e];
				}
				if( out != y ) {
					reinterpret_cast<float4*>( y )[i] = make_float4( centred[0], centred[1], centred[2], centred[3] );
				}
			}
			reinterpret_cast<float4*>( out )[i] = make_float4( result[0], result[1], result[2], result[3] );
		}
	}
}

// The passes of CDnnSimpleGradientSolver::TrainLayer over one parameter blob ( NeoML/src/Dnn/DnnSolver.cpp:481-507 ):
// history *= moment; history += gradient * rate; with L2 regularisation history += parameters * decay; parameters += history
__global__ __launch_bounds__( 256 ) void momentumChainKernel( float* parameters, const float* gradient, float* history,
	const float* moment, const float* rate, const float* decay, int quads )
{
	CMulValueOp<float> byMoment; byMoment.Ptr = moment; byMoment.prepare();
	CMultiplyAndAddOp step; step.Ptr = rate; step.prepare();
	CMultiplyAndAddOp regularise; regularise.Ptr = decay != nullptr ? decay : rate; regularise.prepare();
	const CAddOp<float> sum;
	const int base = blockIdx.x * ( 256 * KnownQuads ) + threadIdx.x;
	float4 p[KnownQuads], g[KnownQuads], h[KnownQuads];
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
			p[u] = reinterpret_cast<const float4*>( parameters )[i];
			g[u] = reinterpret_cast<const float4*>( gradient )[i];
			h[u] = reinterpret_cast<const float4*>( history )[i];
		}
	}
#pragma unroll
	for( int u = 0; u < KnownQuads; ++u ) {
		const int i = base + u * 256;
		if( i < quads ) {
			const float pv[4] = { p[u].x, p[u].y, p[u].z, p[u].w };
			const float gv[4] = { g[u].x, g[u].y, g[u].z, g[u].w };
			float hv[4] = { h[u].x, h[u].y, h[u].z, h[u].w };
			float moved[4];
#pragma unroll
			for( int e = 0; e < 4; ++e ) {
				hv[e] = byMoment( hv[e], 0.f, 0.f );
				hv[e] = step( hv[e], gv[e], 0.f );
				if( decay != nullptr ) {
					hv[e] = regularise( hv[e], pv[e], 0.f );
				}
				moved[e] = sum( pv[e], hv[e], 0.f );
			}
			reinterpret_cast<float4*>( history )[i] = make_float4( hv[0], hv[1], hv[2], hv[3] );
			reinterpret_cast<float4*>( parameters )[i] = make_float4( moved[0], moved[1], moved[2], moved[3] );
		}
	}
}

template<typename F> static bool isKind( const CTinyOp& op ) { return op.Kind == CKindOf<F, CTinyKinds>::Value; }

// A chain of calls of one count on 16-byte boundaries without barriers: true if it was one of the known sequences ( launched )
static bool launchKnownChain( hipStream_t stream, const CTinyChain& chain )
{
	const CTinyOp* op = chain.Ops;
	const int quads = op[0].Count / 4;
	const dim3 grid( ceilDiv( quads, 256 * KnownQuads ) );
	if( chain.Length == 3 && isKind<CMulValueOp<float>>( op[0] ) && isKind<CSigmoidOp>( op[1] ) && isKind<CMulOp<float>>( op[2] )
		&& op[0].Spread == TS_None && op[2].Spread == TS_None ) {
		const float* x = op[0].In[0];
		float* t = op[0].Out;
		const bool product = ( op[2].In[0] == x && op[2].In[1] == t ) || ( op[2].In[0] == t && op[2].In[1] == x );
		// ( the product may go over x: a thread has read its elements of x before it writes any )
		if( x != t && op[1].In[0] == t && op[1].Out == t && product ) {
			hipLaunchKernelGGL( geluChainKernel, grid, dim3( 256 ), 0, stream, x, t, op[2].Out, op[0].Scalar, quads );
			return true;
		}
		return false;
	}
	if( chain.Length == 4 && isKind<CAddOp<float>>( op[0] ) && isKind<CMulOp<float>>( op[1] ) && isKind<CMulOp<float>>( op[2] )
		&& isKind<CAddOp<float>>( op[3] ) && op[0].Spread == TS_PerRow && op[1].Spread == TS_PerRow && op[2].Spread == TS_PerColumn
		&& op[3].Spread == TS_PerColumn && op[1].Width == op[0].Width && op[2].Width == op[0].Width && op[3].Width == op[0].Width ) {
		float* y = op[0].Out;
		float* out = op[2].Out;
		if( op[1].In[0] == y && op[1].Out == y && op[2].In[0] == y && op[3].In[0] == out && op[3].Out == out ) {
			hipLaunchKernelGGL( normalizeChainKernel<false>, grid, dim3( 256 ), 0, stream, op[0].In[0], y, out, op[0].In[1], op[1].In[1],
				op[2].In[1], op[3].In[1], op[0].Width, quads );
			return true;
		}
		return false;
	}
	if( ( chain.Length == 3 || chain.Length == 4 ) && isKind<CMulValueOp<float>>( op[0] ) && isKind<CMultiplyAndAddOp>( op[1] )
		&& isKind<CAddOp<float>>( op[chain.Length - 1] ) && ( chain.Length == 3 || isKind<CMultiplyAndAddOp>( op[2] ) ) ) {
		const CTinyOp& last = op[chain.Length - 1];
		float* history = op[0].Out;
		float* parameters = last.Out;
		const float* gradient = op[1].In[1];
		bool known = op[0].In[0] == history && op[1].In[0] == history && op[1].Out == history && last.Spread == TS_None
			&& ( ( last.In[0] == parameters && last.In[1] == history ) || ( last.In[0] == history && last.In[1] == parameters ) )
			&& parameters != history && gradient != history && gradient != parameters;
		if( chain.Length == 4 ) {
			known = known && op[2].In[0] == history && op[2].In[1] == parameters && op[2].Out == history;
		}
		if( known ) {
			hipLaunchKernelGGL( momentumChainKernel, grid, dim3( 256 ), 0, stream, parameters, gradient, history, op[0].Scalar, op[1].Scalar,
				chain.Length == 4 ? op[2].Scalar : static_cast<const float*>( nullptr ), quads );
			return true;
		}
		return false;
	}
	if( chain.Length == 2 && isKind<CAddOp<float>>( op[0] ) && isKind<CMulOp<float>>( op[1] ) && op[0].Spread == TS_PerRow
		&& op[1].Spread == TS_None ) {
		float* y = op[0].Out;
		if( op[1].In[0] == y && op[1].In[1] == y && op[1].Out == y ) {
			hipLaunchKernelGGL( normalizeChainKernel<true>, grid, dim3( 256 ), 0, stream, op[0].In[0], y, y, op[0].In[1],
				static_cast<const float*>( nullptr ), static_cast<const float*>( nullptr ), static_cast<const float*>( nullptr ),
				op[0].Width, quads );
			return true;
		}
	}
	return false;
}

static bool launchTinyChain( hipStream_t stream, CTinyQueue& queue )
{
	CTinyChain& chain = queue.Chain;
	if( chain.Length == 0 ) {
		return false;
	}
	// ( a call that nothing has joined goes out as the launch it would have been on any other stream: the large ones for
	// their kernels' rates, the small ones because a chain's launch takes 5 us where theirs takes 4 )
	if( chain.Length == 1 && ( chain.Ops[0].Spread != TS_None ? queue.FirstSpreadAlone != nullptr : queue.FirstAlone != nullptr ) ) {
		const CTinyOp op = chain.Ops[0];
		chain.Length = 0;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		if( op.Spread != TS_None ) {
			queue.FirstSpreadAlone( stream, op.Kind == CKindOf<CMulOp<float>, CTinyKinds>::Value, op.Spread, op.In[0], op.In[1], op.Out,
				op.Count / op.Width, op.Width );
		} else {
			queue.FirstAlone( stream, op );
		}
		return true;
	}
	bool barrier = false, quads = true, oneCount = true;
	int longest = 0;
	for( int k = 0; k < chain.Length; ++k ) {
		CTinyOp& op = chain.Ops[k];
		op.Dead = 0;
		barrier = barrier || op.Barrier != 0;
		oneCount = oneCount && op.Count == chain.Ops[0].Count;
		longest = op.Count > longest ? op.Count : longest;
		quads = quads && op.Count == chain.Ops[0].Count && op.Count % 4 == 0 && isAligned16( op.Out )
			&& isAligned16( op.In[0] ) && isAligned16( op.In[1] ) && isAligned16( op.In[2] )
			&& ( op.Spread == TS_None || op.Width % 4 == 0 );
	}
	if( !barrier && oneCount ) {
		// results that a later call overwrites before anything reads them from memory: the kernel's thread takes an operand from
		// a register if the call in front wrote it, or if it is what the first call read ( runStraightChain )
		const float* held = chain.Ops[0].In[0];
		for( int k = 0; k + 1 < chain.Length; ++k ) {
			const float* out = chain.Ops[k].Out;
			for( int j = k + 1; j < chain.Length; ++j ) {
				const CTinyOp& later = chain.Ops[j];
				bool readsFromMemory = false;
				for( int i = 0; i < 3; ++i ) {
					readsFromMemory = readsFromMemory || ( later.In[i] == out && j != k + 1 && out != held );
				}
				if( readsFromMemory ) {
					break;
				}
				if( later.Out == out ) {
					chain.Ops[k].Dead = 1;
					break;
				}
			}
		}
	}
	if( !barrier && quads && longest > TinyOpMaxCount ) {
		if( !launchKnownChain( stream, chain ) ) {
			chain.Straight = 4;
			chain.Blocks = ceilDiv( longest / 4, QuadThreads * QuadsPerThread );
			hipLaunchKernelGGL( quadChainKernel, dim3( chain.Blocks ), dim3( QuadThreads ), 0, stream, chain );
		}
		chain.Length = 0;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		return true;
	}
	// one workgroup with barriers, or a thread per element of the longest call ( workgroups of 64, 256 and 1024 threads take
	// the same 4.6 us for four calls over 8192 elements )
	constexpr int StraightThreads = 256;
	chain.Straight = barrier ? 0 : 1;
	chain.Blocks = barrier ? 1 : ceilDiv( longest, StraightThreads );
	hipLaunchKernelGGL( tinyChainKernel, dim3( chain.Blocks ), dim3( barrier ? TinyThreads : StraightThreads ), 0, stream, chain );
	chain.Length = 0;
	__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

// result[r] = tail( sum_c matrix[r][c] ): a wavefront per row ( sumColumnsKernel of blas_ops.hip, with the same order of
// additions ), then the calls of the tail on the row's value, each with the functor and the device scalar of its own launch
// ( PRODUCER 1: the matrix is first + second, 2: it is ( first + second[row] )^2; written on the way )
template<int PRODUCER>
__global__ __launch_bounds__( 256 )
void sumColumnsTailKernel( float* result, const float* matrix, const float* first, const float* second, float* sum, int height, int width,
	int vec, const CTinyChain tail )
{
	// ( a square must be rounded before it is added to its neighbour, as the separate launches' stored values are )
#pragma clang fp contract( off )
	const int row = blockIdx.x * 4 + ( threadIdx.x >> 6 );
	if( row >= height ) {
		return;
	}
	const int lane = threadIdx.x & 63;
	const long long offset = static_cast<long long>( row ) * width;
	const float* p = matrix + offset;
	const float shift = PRODUCER == 2 ? second[row] : 0.f;
	float s = 0.f;
	if( vec ) {
		const int w4 = width >> 2;
		for( int i = lane; i < w4; i += 64 ) {
			float4 v;
			if( PRODUCER == 1 ) {
				const float4 x = reinterpret_cast<const float4*>( first + offset )[i];
				const float4 y = reinterpret_cast<const float4*>( second + offset )[i];
				v = make_float4( x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w );
				reinterpret_cast<float4*>( sum + offset )[i] = v;
			} else if( PRODUCER == 2 ) {
				const float4 x = reinterpret_cast<const float4*>( first + offset )[i];
				const float4 c = make_float4( x.x + shift, x.y + shift, x.z + shift, x.w + shift );
				v = make_float4( c.x * c.x, c.y * c.y, c.z * c.z, c.w * c.w );
				reinterpret_cast<float4*>( sum + offset )[i] = v;
			} else {
				v = reinterpret_cast<const float4*>( p )[i];
			}
			s += ( v.x + v.y ) + ( v.z + v.w );
		}
	} else {
		for( int i = lane; i < width; i += 64 ) {
			float v;
			if( PRODUCER == 1 ) {
				v = first[offset + i] + second[offset + i];
				sum[offset + i] = v;
			} else if( PRODUCER == 2 ) {
				const float c = first[offset + i] + shift;
				v = c * c;
				sum[offset + i] = v;
			} else {
				v = p[i];
			}
			s += v;
		}
	}
	s = waveReduceSum( s );
	if( lane == 0 ) {
		const float none = 0.f;
		for( int k = 0; k < tail.Length; ++k ) {
			const CTinyOp& op = tail.Ops[k];
			const float scalar = op.Scalar != nullptr ? *op.Scalar : 0.f;
			float next = 0.f;
			CTinyApply<CTinyKinds>::template Run<1>( op.Kind, op, scalar, &s, &none, &none, &next );
			s = next;
		}
		result[row] = s;
	}
}

// what the queue holds: the product that waits for its successor ( then nothing else is queued ), or a chain
static bool launchPending( hipStream_t stream, CTinyQueue& queue )
{
	if( queue.ColumnSum.Pending ) {
		const CPendingColumnSum sum = queue.ColumnSum;
		queue.ColumnSum.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		CTinyChain& tail = queue.Chain; // ( calls in place over the sums, nothing else: deferEltwise sees to that )
		const int vec = ( sum.Width % 4 == 0 && isAligned16( sum.Matrix ) && isAligned16( sum.AddFirst ) && isAligned16( sum.AddSecond )
			&& isAligned16( sum.SquareOf ) ) ? 1 : 0;
		if( sum.AddFirst != nullptr ) {
			hipLaunchKernelGGL( sumColumnsTailKernel<1>, dim3( ceilDiv( sum.Height, 4 ) ), dim3( 256 ), 0, stream, sum.Result, sum.Matrix,
				sum.AddFirst, sum.AddSecond, const_cast<float*>( sum.Matrix ), sum.Height, sum.Width, vec, tail );
		} else if( sum.SquareOf != nullptr ) {
			hipLaunchKernelGGL( sumColumnsTailKernel<2>, dim3( ceilDiv( sum.Height, 4 ) ), dim3( 256 ), 0, stream, sum.Result, sum.Matrix,
				sum.SquareOf, sum.SquareShift, const_cast<float*>( sum.Matrix ), sum.Height, sum.Width, vec, tail );
		} else {
			hipLaunchKernelGGL( sumColumnsTailKernel<0>, dim3( ceilDiv( sum.Height, 4 ) ), dim3( 256 ), 0, stream, sum.Result, sum.Matrix,
				static_cast<const float*>( nullptr ), static_cast<const float*>( nullptr ), static_cast<float*>( nullptr ), sum.Height,
				sum.Width, vec, tail );
		}
		if( tail.Length > 0 ) {
			tail.Length = 0;
			__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		}
		return true;
	}
	if( queue.Product.Pending ) {
		const CPendingProduct p = queue.Product;
		queue.Product.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		// ( a launch that fails leaves its message with nhGetLastError and its HIP error to the next launch check )
		( void )matMulNT( stream, p.A, p.Lda, p.B, p.Ldb, p.C, p.Ldc, p.M, p.N, p.K, 1, 0, 0, 0, nullptr, false );
		return true;
	}
	if( queue.Convolution.Pending ) {
		const CPendingConvolution c = queue.Convolution;
		queue.Convolution.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		const CFusedActivation none = { NH_ACT_NONE, 0.f };
		( void )launchDeferredConvolution( stream, c.Channelwise, c.Desc, c.Source, c.Filter, c.FreeTerm, c.Result, none );
		return true;
	}
	if( queue.Batched.Pending ) {
		const CPendingBatched p = queue.Batched;
		queue.Batched.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		( void )launchBatched( stream, p, nullptr, nullptr );
		return true;
	}
	if( queue.Padding.Pending ) {
		const CPendingPadding p = queue.Padding;
		queue.Padding.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		( void )launchPadding( stream, p );
		return true;
	}
	if( queue.Sum.Pending ) {
		const CPendingSum sum = queue.Sum;
		queue.Sum.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
		( void )launchPlainSum( stream, sum );
		return true;
	}
	return launchTinyChain( stream, queue );
}

bool flushTinyOps( hipStream_t stream )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	return found != tinyQueues().end() && launchPending( stream, found->second );
}

void flushAllTinyOps()
{
	if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) == 0 ) {
		return;
	}
	int current = 0;
	if( hipGetDevice( &current ) != hipSuccess ) {
		( void )hipGetLastError();
		return;
	}
	int active = current;
	std::pair<int, hipStream_t> launched[16];
	int launchedCount = 0;
	{
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		for( auto& entry : tinyQueues() ) {
			if( entry.second.Chain.Length == 0 && !entry.second.LaunchWaits() ) {
				continue;
			}
			if( entry.first.first != active ) {
				if( hipSetDevice( entry.first.first ) != hipSuccess ) {
					( void )hipGetLastError();
					continue;
				}
				active = entry.first.first;
			}
			if( launchPending( entry.first.second, entry.second ) && launchedCount < 16 ) {
				launched[launchedCount++] = entry.first;
			}
		}
	}
	if( __atomic_load_n( &lstmPartnersAwaited, __ATOMIC_RELAXED ) != 0 ) {
		for( int i = 0; i < launchedCount; ++i ) {
			if( launched[i].first != active ) {
				if( hipSetDevice( launched[i].first ) != hipSuccess ) {
					( void )hipGetLastError();
					continue;
				}
				active = launched[i].first;
			}
			noteStreamUse( launched[i].second );
		}
	}
	if( active != current ) {
		( void )hipSetDevice( current );
	}
}

// the stream is going away ( drained by the caller ): a later stream may be handed the same handle
void releaseTinyQueue( hipStream_t stream )
{
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found != tinyQueues().end() ) {
		launchPending( stream, found->second );
		if( found->second.Enabled ) {
			__atomic_fetch_sub( &tinyDeferringStreams, 1, __ATOMIC_RELAXED );
		}
		tinyQueues().erase( found );
	}
}

bool deferProduct( nhStream s, const float* a, int lda, const float* b, int ldb, float* c, int ldc, int M, int N, int K )
{
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || M <= 0 || N <= 0 || K <= 0 || ldc != N ) {
		return false;
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() )
	{
		return false;
	}
	CPendingProduct& p = found->second.Product;
	p.Pending = true;
	p.A = a; p.Lda = lda; p.B = b; p.Ldb = ldb; p.C = c; p.Ldc = ldc; p.M = M; p.N = N; p.K = K;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

bool fusePendingProduct( nhStream s, const float* matrix, float* result, int height, int width, const float* vector, int* rc )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	CPendingProduct p;
	{
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto found = tinyQueues().find( std::make_pair( device, stream ) );
		if( found == tinyQueues().end() || !found->second.Product.Pending ) {
			return false;
		}
		p = found->second.Product;
		if( matrix != p.C || result != p.C || height != p.M || width != p.N || vector == nullptr ) {
			return false; // ( the caller's own launch sends the product out first, as it was asked for )
		}
		found->second.Product.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	}
	*rc = matMulNT( stream, p.A, p.Lda, p.B, p.Ldb, p.C, p.Ldc, p.M, p.N, p.K, 1, 0, 0, 0, vector, false );
	if( __atomic_load_n( &lstmPartnersAwaited, __ATOMIC_RELAXED ) != 0 ) {
		noteStreamUse( stream );
	}
	return true;
}

bool deferColumnSum( nhStream s, float* result, const float* matrix, int height, int width )
{
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || result == nullptr || matrix == nullptr || height <= 0
		|| width <= 0 ) {
		return false;
	}
	if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0 ) {
		// a sum of two matrices that waits on the stream, and these are the sums of its rows: the two wait on as one
		int current = 0;
		if( hipGetDevice( &current ) != hipSuccess ) {
			( void )hipGetLastError();
			return false;
		}
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto waiting = tinyQueues().find( std::make_pair( current, reinterpret_cast<hipStream_t>( s ) ) );
		if( waiting != tinyQueues().end() && waiting->second.Sum.Pending ) {
			const CPendingSum added = waiting->second.Sum;
			const float* resultEnd = result + height;
			const bool apart = resultEnd <= added.Result || added.Result + added.Count <= result;
			if( added.Result == matrix && static_cast<long long>( added.Count ) == static_cast<long long>( height ) * width && apart ) {
				waiting->second.Sum.Pending = false; // ( one thing waits where one waited: the count of waiting queues stays )
				CPendingColumnSum& sum = waiting->second.ColumnSum;
				sum.Pending = true;
				sum.Result = result; sum.Matrix = matrix; sum.Height = height; sum.Width = width;
				sum.AddFirst = added.First; sum.AddSecond = added.Second;
				sum.SquareOf = nullptr; sum.SquareShift = nullptr;
				return true;
			}
		}
		if( waiting != tinyQueues().end() && !waiting->second.LaunchWaits() && waiting->second.Chain.Length == 2 ) {
			// the chain "matrix = source + value per row; matrix *= matrix" waits, and these are the sums of that matrix's rows
			CTinyChain& chain = waiting->second.Chain;
			const CTinyOp& centre = chain.Ops[0];
			const CTinyOp& square = chain.Ops[1];
			const float* resultEnd = result + height;
			const long long count = static_cast<long long>( height ) * width;
			const bool apart = ( resultEnd <= centre.Out || centre.Out + count <= result )
				&& ( resultEnd <= centre.In[0] || centre.In[0] + count <= result )
				&& ( resultEnd <= centre.In[1] || centre.In[1] + height <= result );
			if( centre.Kind == CKindOf<CAddOp<float>, CTinyKinds>::Value && square.Kind == CKindOf<CMulOp<float>, CTinyKinds>::Value
				&& centre.Spread == TS_PerRow && square.Spread == TS_None && centre.Width == width && centre.Count == count
				&& square.Count == count && centre.Out == matrix && square.In[0] == matrix && square.In[1] == matrix && square.Out == matrix
				&& centre.Barrier == 0 && square.Barrier == 0 && apart ) {
				CPendingColumnSum& sum = waiting->second.ColumnSum;
				sum.Pending = true;
				sum.Result = result; sum.Matrix = matrix; sum.Height = height; sum.Width = width;
				sum.AddFirst = nullptr; sum.AddSecond = nullptr;
				sum.SquareOf = centre.In[0]; sum.SquareShift = centre.In[1];
				chain.Length = 0; // ( one thing waits where one waited )
				return true;
			}
		}
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() ) {
		return false;
	}
	CPendingColumnSum& sum = found->second.ColumnSum;
	sum.Pending = true;
	sum.Result = result; sum.Matrix = matrix; sum.Height = height; sum.Width = width;
	sum.AddFirst = nullptr; sum.AddSecond = nullptr;
	sum.SquareOf = nullptr; sum.SquareShift = nullptr;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

bool deferPadding( nhStream s, const CPendingPadding& padding )
{
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 ) {
		return false;
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() ) {
		return false;
	}
	found->second.Padding = padding;
	found->second.Padding.Pending = true;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

// BlobMaxPooling ( no indices ) asks whether it is the call a padded image waits for. true: both have been launched as one.
bool fusePendingPadding( nhStream s, const nhPoolingDesc& d, const float* source, float* result, int* rc )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Padding.Pending || found->second.Padding.To != source ) {
		return false; // ( the caller's own launch sends the padding out first )
	}
	const CPendingPadding p = found->second.Padding;
	found->second.Padding.Pending = false;
	__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	if( launchPaddingWithPooling( stream, p, d, result, rc ) ) {
		return true;
	}
	( void )launchPadding( stream, p ); // ( not a pair for one launch: the padding as it was asked for, the pooling is the caller's )
	return false;
}

bool deferBatchedProduct( nhStream s, int batch, const float* first, int height, int width, const float* second, int secondWidth,
	float* result )
{
	// ( only what the kernel for batches of small products may take: the others have nothing to gain from waiting )
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || batch < 2 || height <= 0 || width <= 0 || width > 256
		|| secondWidth <= 0 || first == nullptr || second == nullptr || result == nullptr
		|| static_cast<long long>( batch ) * height * secondWidth > 0x7fffffffLL ) {
		return false;
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() ) {
		return false;
	}
	CPendingBatched& p = found->second.Batched;
	p.Pending = true;
	p.A = first; p.B = second; p.C = result; p.Batch = batch; p.M = height; p.N = secondWidth; p.K = width;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

// VectorMultiply( first -> result, count, multiplier ) asks whether it is the call a batch of products waits for. true: both
// have been launched as one ( *rc ). false: the caller goes on as usual ( a waiting batch has then been launched by itself if
// this call is over its result but its kernel cannot multiply; otherwise the caller's own launch sends it out first ).
static bool fusePendingBatched( nhStream s, const float* first, float* result, int count, const float* multiplier, int* rc )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	CPendingBatched p;
	{
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto found = tinyQueues().find( std::make_pair( device, stream ) );
		if( found == tinyQueues().end() || !found->second.Batched.Pending ) {
			return false;
		}
		p = found->second.Batched;
		if( first != p.C || result != p.C || multiplier == nullptr
			|| static_cast<long long>( count ) != static_cast<long long>( p.Batch ) * p.M * p.N ) {
			return false;
		}
		found->second.Batched.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	}
	bool scaled = false;
	*rc = launchBatched( stream, p, multiplier, &scaled );
	if( __atomic_load_n( &lstmPartnersAwaited, __ATOMIC_RELAXED ) != 0 ) {
		noteStreamUse( stream );
	}
	return scaled || *rc != NH_OK;
}

static int launchPlainSum( hipStream_t stream, const CPendingSum& sum )
{
	// ( the launch itself: the sum has waited already )
	return launchEltwisePlain<2, float, float>( stream, sum.First, sum.Second, static_cast<const float*>( nullptr ), sum.Result, sum.Count,
		CAddOp<float>() );
}

// a sum of two vectors too large for a chain: it waits for the call behind it
static bool deferSum( nhStream s, const float* first, const float* second, float* result, int count )
{
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || first == nullptr || second == nullptr || result == nullptr ) {
		return false;
	}
	if( __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0 ) {
		// behind calls of the same count that wait as a chain ( a solver's last pass over a blob ) the sum is one more of them
		int current = 0;
		if( hipGetDevice( &current ) != hipSuccess ) {
			( void )hipGetLastError();
			return false;
		}
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto waiting = tinyQueues().find( std::make_pair( current, reinterpret_cast<hipStream_t>( s ) ) );
		if( waiting != tinyQueues().end() && waiting->second.Chain.Length > 0 && waiting->second.Chain.Ops[0].Count == count ) {
			return false;
		}
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() ) {
		return false;
	}
	CPendingSum& sum = found->second.Sum;
	sum.Pending = true;
	sum.First = first; sum.Second = second; sum.Result = result; sum.Count = count;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

static bool fusePendingSum( nhStream s, const float* first, float* result, int count, const float* upperThreshold, int* rc )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	CPendingSum sum;
	{
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto found = tinyQueues().find( std::make_pair( device, stream ) );
		if( found == tinyQueues().end() || !found->second.Sum.Pending ) {
			return false;
		}
		sum = found->second.Sum;
		if( first != sum.Result || result != sum.Result || count != sum.Count ) {
			return false; // ( the caller's own launch sends the sum out first, as it was asked for )
		}
		found->second.Sum.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	}
	CAddReLUOp op; op.Ptr = upperThreshold; op.Threshold = 0;
	*rc = launchEltwise<2, float, float>( s, sum.First, sum.Second, static_cast<const float*>( nullptr ), sum.Result, sum.Count, op );
	return true;
}

bool deferConvolution( nhStream s, bool channelwise, const nhConvDesc& d, const float* source, const float* filter,
	const float* freeTerm, float* result )
{
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || d.batch <= 0 ) {
		return false;
	}
	const hipStream_t stream = toStream( s ); // ( what the stream holds goes out first )
	int device = 0;
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	if( capture != hipStreamCaptureStatusNone ) {
		return false;
	}
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	auto found = tinyQueues().find( std::make_pair( device, stream ) );
	if( found == tinyQueues().end() || !found->second.Enabled || found->second.Chain.Length != 0 || found->second.LaunchWaits() )
	{
		return false;
	}
	CPendingConvolution& c = found->second.Convolution;
	c.Pending = true;
	c.Channelwise = channelwise;
	c.Desc = d;
	c.Source = source; c.Filter = filter; c.FreeTerm = freeTerm; c.Result = result;
	__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	return true;
}

bool fusePendingConvolution( nhStream s, const float* first, float* result, long long count, int activation,
	const float* upperThreshold, int* rc )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	if( hipGetDevice( &device ) != hipSuccess ) {
		( void )hipGetLastError();
		return false;
	}
	CPendingConvolution c;
	{
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto found = tinyQueues().find( std::make_pair( device, stream ) );
		if( found == tinyQueues().end() || !found->second.Convolution.Pending ) {
			return false;
		}
		c = found->second.Convolution;
		const long long resultCount = static_cast<long long>( c.Desc.batch ) * c.Desc.resultHeight * c.Desc.resultWidth * c.Desc.filterCount;
		if( first != c.Result || result != c.Result || count != resultCount || ( activation == NH_ACT_RELU && upperThreshold == nullptr ) ) {
			return false; // ( the caller's own launch sends the convolution out first, as it was asked for )
		}
		found->second.Convolution.Pending = false;
		__atomic_fetch_sub( &tinyChainsPending, 1, __ATOMIC_RELAXED );
	}
	const CFusedActivation act = { activation, 0.f, activation == NH_ACT_RELU ? upperThreshold : nullptr };
	*rc = launchDeferredConvolution( stream, c.Channelwise, c.Desc, c.Source, c.Filter, c.FreeTerm, c.Result, act );
	if( __atomic_load_n( &lstmPartnersAwaited, __ATOMIC_RELAXED ) != 0 ) {
		noteStreamUse( stream );
	}
	return true;
}

struct CFloatRange {
	const float* Lo = nullptr;
	const float* Hi = nullptr;
};
// the ranges share elements without beginning at the same one
static bool rangesClash( const CFloatRange& x, const CFloatRange& y )
{
	return x.Lo != nullptr && y.Lo != nullptr && x.Lo != y.Lo && x.Lo < y.Hi && y.Lo < x.Hi;
}
static bool rangesTouch( const CFloatRange& x, const CFloatRange& y )
{
	return x.Lo != nullptr && y.Lo != nullptr && x.Lo < y.Hi && y.Lo < x.Hi;
}

template<typename F, typename = void> struct CHasScalar : std::false_type {};
template<typename F> struct CHasScalar<F, decltype( static_cast<void>( std::declval<F>().Ptr ) )> : std::true_type {};

// the device scalar a functor reads when the kernel starts, if it has one
template<typename F> static auto scalarOf( const F& f, int ) -> decltype( static_cast<const float*>( f.Ptr ) ) { return f.Ptr; }
template<typename F> static const float* scalarOf( const F&, long ) { return nullptr; }

// what a call reads of its spread operand
static CFloatRange spreadRange( const CTinyOp& op )
{
	CFloatRange range;
	range.Lo = op.In[1];
	range.Hi = op.In[1] + ( op.Spread == TS_PerRow ? op.Count / op.Width : op.Width );
	return range;
}

template<int NIN, typename F> static void launchTinyOpAlone( hipStream_t stream, const CTinyOp& op )
{
	F f;
	__builtin_memcpy( &f, op.Functor, sizeof( F ) );
	// ( a launch that fails leaves its HIP error to the next launch check )
	( void )launchEltwisePlain<NIN, float, float, F>( stream, op.In[0], op.In[1], op.In[2], op.Out, op.Count, f );
}

template<int NIN, typename TIn, typename TOut, typename F>
static bool deferEltwise( nhStream s, const TIn* a, const TIn* b, const TIn* c, TOut* out, int n, const F& f, int spread, int width,
	CSpreadAlone spreadAlone )
{
	if constexpr( std::is_same<TIn, float>::value && std::is_same<TOut, float>::value && CKindOf<F, CTinyKinds>::Value >= 0 ) {
		if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 ) {
			return false;
		}
		const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
		int device = 0;
		hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
		if( hipGetDevice( &device ) != hipSuccess || hipStreamIsCapturing( stream, &capture ) != hipSuccess ) {
			( void )hipGetLastError();
			return false;
		}
		if( capture != hipStreamCaptureStatusNone ) {
			return false; // the recording ends outside this library: nothing may be left behind
		}
		std::lock_guard<std::recursive_mutex> guard( tinyLock );
		auto found = tinyQueues().find( std::make_pair( device, stream ) );
		if( found == tinyQueues().end() || !found->second.Enabled ) {
			return false;
		}
		if( found->second.ColumnSum.Pending ) {
			// row sums wait: a call with one operand, in place over exactly those sums, joins their tail
			const CPendingColumnSum& sum = found->second.ColumnSum;
			const float* own = scalarOf( f, 0 );
			const bool tail = NIN == 1 && spread == TS_None && a == out && out == sum.Result && n == sum.Height
				&& found->second.Chain.Length < TinyChainMax && ( own == nullptr || own + 1 <= out || own >= out + n );
			if( !tail ) {
				launchPending( stream, found->second );
			}
		} else if( found->second.LaunchWaits() ) {
			launchPending( stream, found->second ); // ( a launch that waited for its successor: this call is not the one )
		}
		CTinyQueue& queue = found->second;
		CTinyChain& chain = queue.Chain;
		if( chain.Length > 0 && ( n > TinyWideMaxCount || chain.Ops[0].Count > TinyWideMaxCount ) && chain.Ops[0].Count != n ) {
			launchTinyChain( stream, queue ); // ( a chain with a call that large holds calls of one count only )
		}
		if( chain.Length == TinyChainMax ) {
			launchTinyChain( stream, queue );
		}
		CTinyOp op = CTinyOp();
		op.In[0] = NIN >= 1 ? a : nullptr;
		op.In[1] = NIN >= 2 ? b : nullptr;
		op.In[2] = NIN >= 3 ? c : nullptr;
		op.Out = out;
		op.Count = n;
		op.Kind = static_cast<short>( CKindOf<F, CTinyKinds>::Value );
		op.Spread = spread;
		op.Width = width;
		__builtin_memcpy( op.Functor, &f, sizeof( F ) );
		// what the calls in front have to do with this one ( reads[4]: a spread operand, read by many threads like the scalar )
		CFloatRange reads[5], writes;
		for( int i = 0; i < 3; ++i ) {
			if( op.In[i] != nullptr && ( i != 1 || spread == TS_None ) ) {
				reads[i].Lo = op.In[i];
				reads[i].Hi = op.In[i] + n;
			}
		}
		if( spread != TS_None ) {
			reads[4] = spreadRange( op );
		}
		const float* scalar = scalarOf( f, 0 );
		// ( a functor with a device scalar is { pointer, value }: tinyChainKernel puts the value it has fetched behind the pointer )
		static_assert( std::is_same<decltype( scalarOf( f, 0 ) ), const float*>::value, "scalars of chained calls are floats" );
		if constexpr( CHasScalar<F>::value ) {
			static_assert( sizeof( F ) == 16 && offsetof( F, Ptr ) == 0, "layout of a functor with a device scalar" );
		} else {
			static_assert( sizeof( F ) != 16, "only functors with a device scalar are 16 bytes" );
		}
		op.Scalar = scalar;
		if( scalar != nullptr ) {
			reads[3].Lo = scalar;
			reads[3].Hi = scalar + 1;
		}
		writes.Lo = out;
		writes.Hi = out + n;
		bool barrier = false, wide = n > TinyOpMaxCount;
		for( int k = 0; k < chain.Length; ++k ) {
			wide = wide || chain.Ops[k].Count > TinyOpMaxCount;
		}
		for( int k = 0; k < chain.Length && !barrier; ++k ) {
			const CTinyOp& front = chain.Ops[k];
			CFloatRange frontWrites;
			frontWrites.Lo = front.Out;
			frontWrites.Hi = front.Out + front.Count;
			// ( the scalar: read by every thread, so a match of the first element is no excuse )
			barrier = rangesClash( reads[0], frontWrites ) || rangesClash( reads[1], frontWrites ) || rangesClash( reads[2], frontWrites )
				|| rangesTouch( reads[3], frontWrites ) || rangesTouch( reads[4], frontWrites ) || rangesClash( writes, frontWrites );
			for( int i = 0; i < 3 && !barrier; ++i ) {
				if( front.In[i] != nullptr && ( i != 1 || front.Spread == TS_None ) ) {
					CFloatRange frontReads;
					frontReads.Lo = front.In[i];
					frontReads.Hi = front.In[i] + front.Count;
					barrier = rangesClash( writes, frontReads );
				}
			}
			if( !barrier && front.Spread != TS_None ) {
				barrier = rangesTouch( writes, spreadRange( front ) );
			}
			if( !barrier && front.Scalar != nullptr ) {
				CFloatRange frontReads;
				frontReads.Lo = front.Scalar;
				frontReads.Hi = front.Scalar + 1;
				barrier = rangesTouch( writes, frontReads );
			}
		}
		if( barrier && wide ) {
			// a chain with a barrier is one workgroup, too few threads for this many elements: what is in front goes out
			// now, and this call is the first of the next chain
			launchTinyChain( stream, queue );
			barrier = false;
		}
		op.Barrier = barrier ? 1 : 0;
		if( chain.Length == 0 ) {
			__atomic_fetch_add( &tinyChainsPending, 1, __ATOMIC_RELAXED );
			queue.FirstAlone = &launchTinyOpAlone<NIN, F>;
			queue.FirstSpreadAlone = spreadAlone;
		}
		chain.Ops[chain.Length] = op;
		++chain.Length;
		return true;
	} else {
		( void )s; ( void )a; ( void )b; ( void )c; ( void )out; ( void )n; ( void )f; ( void )spread; ( void )width; ( void )spreadAlone;
		return false;
	}
}

bool deferSpreadOp( nhStream s, bool multiply, int spread, const float* matrix, const float* vector, float* result, int height, int width,
	CSpreadAlone alone )
{
	const long long count = static_cast<long long>( height ) * width;
	if( __atomic_load_n( &tinyDeferringStreams, __ATOMIC_RELAXED ) == 0 || count <= TinyWideMaxCount || count > 0x7fffffffLL
		|| matrix == nullptr || vector == nullptr || result == nullptr || alone == nullptr
		|| ( spread != TS_PerRow && spread != TS_PerColumn ) ) {
		return false;
	}
	const float* none = nullptr;
	if( multiply ) {
		return deferEltwise<2, float, float, CMulOp<float>>( s, matrix, vector, none, result, static_cast<int>( count ), CMulOp<float>(),
			spread, width, alone );
	}
	return deferEltwise<2, float, float, CAddOp<float>>( s, matrix, vector, none, result, static_cast<int>( count ), CAddOp<float>(),
		spread, width, alone );
}

// ---- reductions to one value: one workgroup per 16K elements ------------------------------------------------------
// The workgroups meet in the stream's scratch: each leaves its partial sum there and draws a ticket; the one that draws
// the last ticket adds the partial sums up in a fixed order and only then touches the result ( stores, or adds onto it ).
// So the value does not depend on the order in which the workgroups finish, and a result that lies inside an operand
// is read before it is written, as on the CPU engine. Without scratch ( a capturing stream ): atomic adds onto a
// result that a launch in front has set to zero.

// VEC: 128-bit loads, four of them in flight per thread and operand (both pointers 16-byte aligned); the up to three
// elements behind the last whole vector are added by the first thread.
template<bool DOT, bool VEC, bool STREAM = false>
__global__ __launch_bounds__( 256 ) void sumKernel( const float* a, const float* b, int n, float* result, float* partials,
	unsigned* counter, int addToResult )
{
	__shared__ float part[4];
	__shared__ unsigned ticket;
	float s = 0.f;
	const int stride = gridDim.x * 256;
	const int start = blockIdx.x * 256 + threadIdx.x;
	if( VEC ) {
		// a workgroup reads runs of 32 KB ( eight 128-bit loads in flight per lane ), the workgroups' runs interleaved; with
		// the streaming hint for vectors far beyond the last-level cache. Measured ( 67 M / 268 M floats, us ): runs of 4 KB
		// and four loads in flight 55 / 216, one contiguous piece per workgroup 59 / 175, these runs 58 / 172 ( 6.2 TB/s )
		const int n4 = n >> 2;
		const float4* a4 = reinterpret_cast<const float4*>( a );
		const float4* b4 = reinterpret_cast<const float4*>( b );
		constexpr int Unroll = 8;
		constexpr int Run = Unroll * 256;
		float acc[Unroll] = {};
		const int wholeRuns = n4 / Run;
		for( int run = blockIdx.x; run < wholeRuns; run += gridDim.x ) {
			const int i = run * Run + threadIdx.x;
			float4 va[Unroll], vb[Unroll];
#pragma unroll
			for( int j = 0; j < Unroll; ++j ) {
				va[j] = STREAM ? loadStreaming( a4 + i + j * 256 ) : a4[i + j * 256];
				if( DOT ) {
					vb[j] = STREAM ? loadStreaming( b4 + i + j * 256 ) : b4[i + j * 256];
				}
			}
#pragma unroll
			for( int j = 0; j < Unroll; ++j ) {
				acc[j] += DOT ? ( va[j].x * vb[j].x + va[j].y * vb[j].y ) + ( va[j].z * vb[j].z + va[j].w * vb[j].w )
					: ( va[j].x + va[j].y ) + ( va[j].z + va[j].w );
			}
		}
		// what is left behind the whole runs: less than one run, shared by all workgroups
		for( int i = wholeRuns * Run + start; i < n4; i += stride ) {
			const float4 va = a4[i];
			if( DOT ) {
				const float4 vb = b4[i];
				acc[0] += ( va.x * vb.x + va.y * vb.y ) + ( va.z * vb.z + va.w * vb.w );
			} else {
				acc[0] += ( va.x + va.y ) + ( va.z + va.w );
			}
		}
		s = ( ( acc[0] + acc[1] ) + ( acc[2] + acc[3] ) ) + ( ( acc[4] + acc[5] ) + ( acc[6] + acc[7] ) );
		if( start == 0 ) {
			for( int k = n4 << 2; k < n; ++k ) {
				s += DOT ? a[k] * b[k] : a[k];
			}
		}
	} else {
		for( int i = start; i < n; i += stride ) {
			s += DOT ? a[i] * b[i] : a[i];
		}
	}
	s = waveReduceSum( s );
	if( ( threadIdx.x & 63 ) == 0 ) {
		part[threadIdx.x >> 6] = s;
	}
	__syncthreads();
	const float mine = part[0] + part[1] + part[2] + part[3];
	if( partials == nullptr ) {
		if( threadIdx.x == 0 ) {
			atomicAdd( result, mine );
		}
		return;
	}
	if( gridDim.x == 1 ) {
		if( threadIdx.x == 0 ) {
			*result = addToResult ? *result + mine : mine;
		}
		return;
	}
	// ( values cross between workgroups through device-scope accesses, past the L2 of the XCD they run on )
	if( threadIdx.x == 0 ) {
		__hip_atomic_store( reinterpret_cast<unsigned*>( partials ) + blockIdx.x, __float_as_uint( mine ), __ATOMIC_RELAXED,
			__HIP_MEMORY_SCOPE_AGENT );
		__builtin_amdgcn_s_waitcnt( 0x0F70 ); // vmcnt( 0 ): the store has been acknowledged
		ticket = __hip_atomic_fetch_add( counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
	}
	__syncthreads();
	if( ticket != gridDim.x - 1 || threadIdx.x >= 64 ) {
		return;
	}
	float total = 0.f;
	for( unsigned i = threadIdx.x; i < gridDim.x; i += 64 ) {
		total += __uint_as_float( __hip_atomic_load( reinterpret_cast<unsigned*>( partials ) + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT ) );
	}
	total = waveReduceSum( total );
	if( threadIdx.x == 0 ) {
		*result = addToResult ? *result + total : total;
		__hip_atomic_store( counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT );
	}
}

template<bool DOT>
static int launchSum( nhStream s, const float* first, const float* second, int vectorSize, float* result, bool addToResult = false )
{
	if( vectorSize == 0 ) {
		return addToResult ? NH_OK : nhVectorFill( s, result, 0.f, 1 );
	}
	NH_REQUIRE( first != nullptr && ( !DOT || second != nullptr ) && result != nullptr );
	int blocks = ceilDiv( vectorSize, 16384 );
	blocks = blocks > 2048 ? 2048 : blocks;
	float* partials = nullptr;
	unsigned* counter = nullptr;
	if( !streamMeetingPlace( toStream( s ), 2048, &partials, &counter ) ) {
		partials = nullptr;
		// a result that lies inside an operand must be read before it is written: zeroing it first would change the
		// operand, so such a call ( rare: a capturing stream and an aliased result ) goes to one workgroup
		const auto inside = [&]( const float* operand ) {
			return operand != nullptr && result >= operand && result < operand + vectorSize;
		};
		if( inside( first ) || ( DOT && inside( second ) ) ) {
			blocks = 1;
		}
		if( blocks == 1 ) {
			partials = result; // ( not used by a single workgroup: only says that it may write the result itself )
		} else if( !addToResult ) {
			const int rc = nhVectorFill( s, result, 0.f, 1 );
			if( rc != NH_OK ) {
				return rc;
			}
		}
	}
	const int add = addToResult ? 1 : 0;
	if( isAligned16( first ) && ( !DOT || isAligned16( second ) ) && static_cast<long long>( vectorSize ) * ( DOT ? 2 : 1 ) >= ( 96LL << 20 ) ) {
		hipLaunchKernelGGL( ( sumKernel<DOT, true, true> ), dim3( blocks ), dim3( 256 ), 0, toStream( s ), first, second, vectorSize, result,
			partials, counter, add );
	} else if( isAligned16( first ) && ( !DOT || isAligned16( second ) ) ) {
		hipLaunchKernelGGL( ( sumKernel<DOT, true> ), dim3( blocks ), dim3( 256 ), 0, toStream( s ), first, second, vectorSize, result, partials,
			counter, add );
	} else {
		hipLaunchKernelGGL( ( sumKernel<DOT, false> ), dim3( blocks ), dim3( 256 ), 0, toStream( s ), first, second, vectorSize, result, partials,
			counter, add );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}

} // namespace nh

using namespace nh;

extern "C" int nhStreamDeferSmallOps( nhStream s, int enable )
{
	const hipStream_t stream = reinterpret_cast<hipStream_t>( s );
	int device = 0;
	NH_HIP( hipGetDevice( &device ) );
	std::lock_guard<std::recursive_mutex> guard( tinyLock );
	CTinyQueue& queue = tinyQueues()[std::make_pair( device, stream )];
	if( ( enable != 0 ) != queue.Enabled ) {
		queue.Enabled = enable != 0;
		if( queue.Enabled ) {
			__atomic_fetch_add( &tinyDeferringStreams, 1, __ATOMIC_RELAXED );
		} else {
			__atomic_fetch_sub( &tinyDeferringStreams, 1, __ATOMIC_RELAXED );
			launchPending( stream, queue );
			NH_LAUNCH_CHECK();
		}
	}
	return NH_OK;
}

#define NH_UNARY( name, Op ) \
	extern "C" int name( nhStream s, const float* first, float* result, int vectorSize ) \
	{ return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, Op() ); }

#define NH_BINARY( name, T, Op ) \
	extern "C" int name( nhStream s, const T* first, const T* second, T* result, int vectorSize ) \
	{ return launchEltwise<2, T, T>( s, first, second, (const T*)nullptr, result, vectorSize, Op() ); }

extern "C" int nhVectorCopy( nhStream s, float* first, const float* second, int vectorSize )
{
	return launchEltwise<1, float, float>( s, second, (const float*)nullptr, (const float*)nullptr, first, vectorSize, CCopyOp<float>() );
}
extern "C" int nhVectorCopyInt( nhStream s, int* first, const int* second, int vectorSize )
{
	return launchEltwise<1, int, int>( s, second, (const int*)nullptr, (const int*)nullptr, first, vectorSize, CCopyOp<int>() );
}
extern "C" int nhVectorFill( nhStream s, float* result, float value, int vectorSize )
{
	CFillOp<float> op; op.Value = value;
	return launchEltwise<0, float, float>( s, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorFillInt( nhStream s, int* result, int value, int vectorSize )
{
	CFillOp<int> op; op.Value = value;
	return launchEltwise<0, int, int>( s, (const int*)nullptr, (const int*)nullptr, (const int*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorFillFromHandle( nhStream s, float* result, int vectorSize, const float* value )
{
	NH_REQUIRE( value != nullptr );
	CFillFromOp<float> op; op.Ptr = value; op.Value = 0;
	return launchEltwise<0, float, float>( s, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorFillFromHandleInt( nhStream s, int* result, int vectorSize, const int* value )
{
	NH_REQUIRE( value != nullptr );
	CFillFromOp<int> op; op.Ptr = value; op.Value = 0;
	return launchEltwise<0, int, int>( s, (const int*)nullptr, (const int*)nullptr, (const int*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorConvertFloatToInt( nhStream s, const float* from, int* to, int vectorSize )
{
	return launchEltwise<1, float, int>( s, from, (const float*)nullptr, (const float*)nullptr, to, vectorSize, CFloatToIntOp() );
}
extern "C" int nhVectorConvertIntToFloat( nhStream s, const int* from, float* to, int vectorSize )
{
	return launchEltwise<1, int, float>( s, from, (const int*)nullptr, (const int*)nullptr, to, vectorSize, CIntToFloatOp() );
}

extern "C" int nhVectorReLU( nhStream s, const float* first, float* result, int vectorSize, const float* upperThreshold )
{
	NH_REQUIRE( upperThreshold != nullptr );
	int rc = NH_OK;
	if( first == result && __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0
		&& ( fusePendingConvolution( s, first, result, vectorSize, NH_ACT_RELU, upperThreshold, &rc )
			|| fusePendingSum( s, first, result, vectorSize, upperThreshold, &rc ) ) )
	{
		return rc; // ( the convolution or the sum that waited for this call took the activation with it )
	}
	CReLUOp op; op.Ptr = upperThreshold; op.Threshold = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorELU( nhStream s, const float* first, float* result, int vectorSize, const float* alpha )
{
	NH_REQUIRE( alpha != nullptr );
	CELUOp op; op.Ptr = alpha; op.Alpha = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorLeakyReLU( nhStream s, const float* first, float* result, int vectorSize, const float* alpha )
{
	NH_REQUIRE( alpha != nullptr );
	CLeakyReLUOp op; op.Ptr = alpha; op.Alpha = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorHardSigmoid( nhStream s, const float* first, float* result, int vectorSize,
	const float* slope, const float* bias )
{
	NH_REQUIRE( slope != nullptr && bias != nullptr );
	CHardSigmoidOp op; op.SlopePtr = slope; op.BiasPtr = bias; op.Slope = 0; op.Bias = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMinMax( nhStream s, const float* first, float* result, int vectorSize,
	const float* minValue, const float* maxValue )
{
	NH_REQUIRE( minValue != nullptr && maxValue != nullptr );
	CMinMaxOp op; op.MinPtr = minValue; op.MaxPtr = maxValue; op.Min = 0; op.Max = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}

extern "C" int nhVectorHSwish( nhStream s, const float* first, float* result, int vectorSize )
{
	// ( in place behind a convolution that waits for its successor: the convolution's launch applies it, as it does a ReLU )
	int rc = NH_OK;
	if( first == result && first != nullptr && __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0
		&& fusePendingConvolution( s, first, result, vectorSize, NH_ACT_HSWISH, nullptr, &rc ) ) {
		return rc;
	}
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, CHSwishOp() );
}
NH_UNARY( nhVectorAbs, CAbsOp )
NH_UNARY( nhVectorHardTanh, CHardTanhOp )
NH_UNARY( nhVectorNeg, CNegOp )
NH_UNARY( nhVectorExp, CExpOp )
NH_UNARY( nhVectorLog, CLogOp )
NH_UNARY( nhVectorErf, CErfOp )
NH_UNARY( nhVectorSqrt, CSqrtOp )
NH_UNARY( nhVectorInv, CInvOp )
NH_UNARY( nhVectorSigmoid, CSigmoidOp )
NH_UNARY( nhVectorTanh, CTanhOp )

NH_UNARY( nhVectorNegLog, CNegLogOp )
NH_BINARY( nhVectorHSwishDiff, float, CHSwishDiffOp )
NH_BINARY( nhVectorSigmoidDiff, float, CSigmoidDiffOp )
NH_BINARY( nhVectorSigmoidDiffOp, float, CSigmoidDiffOutOp )
NH_BINARY( nhVectorTanhDiff, float, CTanhDiffOp )
NH_BINARY( nhVectorTanhDiffOp, float, CTanhDiffOutOp )

extern "C" int nhVectorReLUDiff( nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* upperThreshold )
{
	NH_REQUIRE( upperThreshold != nullptr );
	CReLUDiffOp op; op.Ptr = upperThreshold; op.Threshold = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}

#define NH_BINARY_ALPHA( name, Op ) \
	extern "C" int name( nhStream s, const float* first, const float* second, float* result, int vectorSize, const float* alpha ) \
	{ \
		NH_REQUIRE( alpha != nullptr ); \
		Op op; op.Ptr = alpha; op.Alpha = 0; \
		return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op ); \
	}
NH_BINARY_ALPHA( nhVectorELUDiff, CELUDiffOp )
NH_BINARY_ALPHA( nhVectorELUDiffOp, CELUDiffOutOp )
NH_BINARY_ALPHA( nhVectorLeakyReLUDiff, CLeakyReLUDiffOp )
NH_BINARY( nhVectorHardTanhDiff, float, CHardTanhDiffOp )
NH_BINARY( nhVectorAbsDiff, float, CAbsDiffOp )

extern "C" int nhVectorHardSigmoidDiff( nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* slope, const float* bias )
{
	NH_REQUIRE( slope != nullptr && bias != nullptr );
	CHardSigmoidDiffOp op; op.SlopePtr = slope; op.BiasPtr = bias; op.Slope = op.Low = op.High = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorHardSigmoidDiffOp( nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* slope )
{
	NH_REQUIRE( slope != nullptr );
	CHardSigmoidDiffOutOp op; op.SlopePtr = slope; op.Slope = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorSubValue( nhStream s, const float* first, float value, int reverse, float* result, int vectorSize )
{
	CSubValueOp op; op.Value = value; op.Reverse = reverse;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}

NH_UNARY( nhVectorHinge, CHingeOp )
NH_UNARY( nhVectorSquaredHinge, CSquaredHingeOp )
NH_UNARY( nhVectorHuber, CHuberOp )
NH_UNARY( nhVectorHuberDerivative, CHuberDerivativeOp )
NH_BINARY( nhVectorHingeDiff, float, CHingeDiffOp )
NH_BINARY( nhVectorSquaredHingeDiff, float, CSquaredHingeDiffOp )
extern "C" int nhVectorL1DiffAdd( nhStream s, const float* first, const float* second, float* result, int vectorSize,
	const float* threshold, const float* mult )
{
	NH_REQUIRE( threshold != nullptr && mult != nullptr );
	CL1DiffAddOp op; op.ThresholdPtr = threshold; op.MultPtr = mult; op.Threshold = op.Mult = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}

NH_BINARY( nhVectorEltwiseMax, float, CMaxOp )
NH_BINARY( nhVectorEltwiseMin, float, CMinOp )
extern "C" int nhVectorAdd( nhStream s, const float* first, const float* second, float* result, int vectorSize )
{
	// ( on a stream that puts calls aside a large sum waits for the call behind it: a ReLU over it in place is the same pass )
	if( vectorSize > TinyWideMaxCount && deferSum( s, first, second, result, vectorSize ) ) {
		return NH_OK;
	}
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, CAddOp<float>() );
}
NH_BINARY( nhVectorAddInt, int, CAddOp<int> )
NH_BINARY( nhVectorSub, float, CSubOp<float> )
NH_BINARY( nhVectorSubInt, int, CSubOp<int> )
NH_BINARY( nhVectorEltwiseMultiply, float, CMulOp<float> )
NH_BINARY( nhVectorEltwiseMultiplyInt, int, CMulOp<int> )
NH_BINARY( nhVectorEltwiseNegMultiply, float, CNegMulOp )
NH_BINARY( nhVectorEltwiseDivide, float, CDivOp )

extern "C" int nhVectorEltwiseMultiplyAdd( nhStream s, const float* first, const float* second, float* result, int vectorSize )
{
	return launchEltwise<3, float, float>( s, first, second, result, result, vectorSize, CMulAddOp() );
}

extern "C" int nhVectorAddValue( nhStream s, const float* first, float* result, int vectorSize, const float* addition )
{
	NH_REQUIRE( addition != nullptr );
	CAddValueOp<float> op; op.Ptr = addition; op.Value = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorAddValueInt( nhStream s, const int* first, int* result, int vectorSize, const int* addition )
{
	NH_REQUIRE( addition != nullptr );
	CAddValueOp<int> op; op.Ptr = addition; op.Value = 0;
	return launchEltwise<1, int, int>( s, first, (const int*)nullptr, (const int*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMultiply( nhStream s, const float* first, float* result, int vectorSize, const float* multiplier )
{
	NH_REQUIRE( multiplier != nullptr );
	int rc = NH_OK;
	if( first == result && __atomic_load_n( &tinyChainsPending, __ATOMIC_RELAXED ) != 0
		&& fusePendingBatched( s, first, result, vectorSize, multiplier, &rc ) ) {
		return rc; // ( a batch of products was waiting for this call )
	}
	CMulValueOp<float> op; op.Ptr = multiplier; op.Value = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMultiplyInt( nhStream s, const int* first, int* result, int vectorSize, const int* multiplier )
{
	NH_REQUIRE( multiplier != nullptr );
	CMulValueOp<int> op; op.Ptr = multiplier; op.Value = 0;
	return launchEltwise<1, int, int>( s, first, (const int*)nullptr, (const int*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorNegMultiply( nhStream s, const float* first, float* result, int vectorSize, const float* multiplier )
{
	NH_REQUIRE( multiplier != nullptr );
	CNegMulValueOp op; op.Ptr = multiplier; op.Value = 0;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMultiplyAndAdd( nhStream s, const float* first, const float* second, float* result,
	int vectorSize, const float* mult )
{
	NH_REQUIRE( mult != nullptr );
	CMultiplyAndAddOp op; op.Ptr = mult; op.Mult = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMultiplyAndSub( nhStream s, const float* first, const float* second, float* result,
	int vectorSize, const float* mult )
{
	NH_REQUIRE( mult != nullptr );
	CMultiplyAndSubOp op; op.Ptr = mult; op.Mult = 0;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}

extern "C" int nhVectorSum( nhStream s, const float* first, int vectorSize, float* result )
{
	NH_REQUIRE( vectorSize >= 0 && result != nullptr );
	return launchSum<false>( s, first, nullptr, vectorSize, result );
}
extern "C" int nhVectorDotProduct( nhStream s, const float* first, const float* second, int vectorSize, float* result )
{
	NH_REQUIRE( vectorSize >= 0 && result != nullptr );
	return launchSum<true>( s, first, second, vectorSize, result );
}

// ---- comparisons, selections, powers, masked gradients: the element-wise members that losses, ONNX-style operators
// ---- and the automatic differentiation of NeoML call (semantics: src/CPU/CpuMathEngineVectorMath.cpp and
// ---- src/CPU/x86/CpuX86MathEngineVectorMath.cpp, lines cited per functor) ------------------------------------------

namespace nh {

struct CFilterSmallOp { // x86/CpuX86MathEngineVectorMath.cpp:99-126: kept when x >= t or x <= -t
	float Threshold;
	__device__ void prepare() {}
	__device__ float operator()( float a, float, float ) const { return ( a >= Threshold || a <= -Threshold ) ? a : 0.f; }
};
struct CEqualToFloatOp : CNoScalar { __device__ float operator()( int a, int b, int ) const { return a == b ? 1.f : 0.f; } }; // x86:166
struct CEqualValueOp { // x86:199
	const int* Ptr; int Value;
	__device__ void prepare() { Value = *Ptr; }
	__device__ float operator()( int a, int, int ) const { return a == Value ? 1.f : 0.f; }
};
struct CMaxValueOp { // CpuMathEngineVectorMath.cpp:551
	float Value;
	__device__ void prepare() {}
	__device__ float operator()( float a, float, float ) const { return a >= Value ? a : Value; }
};
struct CBernulliKLOp { // x86:980-1025: -t / e + ( 1 - t ) / ( 1 - e ), cut to [-10, 10] (min first, as the SSE code does)
	const float* Ptr; float Target;
	__device__ void prepare() { Target = *Ptr; }
	__device__ float operator()( float e, float, float ) const
	{
		float d = -Target / e + ( 1.f - Target ) / ( 1.f - e );
		d = d < 10.f ? d : 10.f;   // _mm_min_ps( d, 10 ): the second operand when either is NaN
		return d > -10.f ? d : -10.f;
	}
};
struct CDivIntOp : CNoScalar { __device__ int operator()( int a, int b, int ) const { return b != 0 ? a / b : 0; } }; // :814 ( a zero divisor traps there )
struct CEltwisePowerOp : CNoScalar { __device__ float operator()( float a, float b, float ) const { return b == 1.f ? a : powf( a, b ); } }; // x86:1277
struct CPowerOp { // x86/CpuX86MathEngineVectorMathMkl.cpp:129-153
	float Exponent;
	__device__ void prepare() {}
	__device__ float operator()( float a, float, float ) const { return powf( a, Exponent ); }
};
struct CPowerDiffOp { // x86:1522-1595: second * exponent * first ^ Power
	float Exponent, Power;
	__device__ void prepare() {}
	__device__ float operator()( float a, float b, float ) const { return b * ( Exponent * powf( a, Power ) ); }
};
struct CNotOp : CNoScalar { __device__ int operator()( int a, int, int ) const { return a == 0 ? 1 : 0; } };              // x86:1648
struct CNotNegativeOp : CNoScalar { __device__ float operator()( int a, int, int ) const { return a >= 0 ? 1.f : 0.f; } }; // x86:1677
template<typename TIn, typename TOut> struct CLessOp : CNoScalar { // :688-760
	__device__ TOut operator()( TIn a, TIn b, TIn ) const { return static_cast<TOut>( a < b ? 1 : 0 ); }
};
struct CLessValueOp { // :713-741; Reverse: value < x
	float Value; int Reverse;
	__device__ void prepare() {}
	__device__ float operator()( float a, float, float ) const { return ( Reverse ? Value < a : a < Value ) ? 1.f : 0.f; }
};
template<typename TIn> struct CEqualToIntOp : CNoScalar { __device__ int operator()( TIn a, TIn b, TIn ) const { return a == b ? 1 : 0; } }; // :764-786
// first != 0 ? second : third, on the 32-bit patterns (serves the float and the int overload, :788-812)
struct CWhereOp : CNoScalar { __device__ int operator()( int a, int b, int c ) const { return a != 0 ? b : c; } };

// result[i][j] = f( first[i], grad[i][j] ): the gradient forms whose condition is one value per row of the gradient
// ( firstSize = gradHeight == 1 ? gradWidth : gradHeight rows of gradSize = gradHeight == 1 ? 1 : gradWidth values )
template<typename F>
__global__ __launch_bounds__( 256 )
void rowConditionKernel( const float* first, const float* grad, float* result, long long total, int gradSize, F f )
{
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		result[i] = f( first[i / gradSize], grad[i] );
	}
}

struct CRowAbsDiff { __device__ float operator()( float x, float g ) const { return x > 0.f ? g : -g; } };              // :516-549
struct CRowMaxDiff { float Value; __device__ float operator()( float x, float g ) const { return x < Value ? 0.f : g; } }; // :567-589
struct CRowLogDiff { // :591-619
	__device__ float operator()( float x, float g ) const { return ( -FLT_MIN <= x && x <= FLT_MIN ) ? 0.f : g / x; }
};
struct CRowMinMaxDiff { // :649-686
	const float* MinPtr; const float* MaxPtr;
	__device__ float operator()( float x, float g ) const { return ( x < *MinPtr || x > *MaxPtr ) ? 0.f : g; }
};

template<typename F>
static int launchRowCondition( nhStream s, const float* first, const float* grad, float* result, int gradHeight, int gradWidth, F f )
{
	NH_REQUIRE( gradHeight > 0 && gradWidth > 0 && first != nullptr && grad != nullptr && result != nullptr );
	const int gradSize = gradHeight == 1 ? 1 : gradWidth;
	const long long total = static_cast<long long>( gradHeight ) * gradWidth;
	const long long blocks = ( total + 255 ) / 256;
	hipLaunchKernelGGL( rowConditionKernel<F>, dim3( static_cast<unsigned>( blocks > 8192 ? 8192 : blocks ) ), dim3( 256 ), 0, toStream( s ),
		first, grad, result, total, gradSize, f );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

__global__ __launch_bounds__( 256 )
void maxWithIndexKernel( const float* candidate, float* result, int* indices, int index, int n )
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if( i < n && candidate[i] > result[i] ) {
		result[i] = candidate[i];
		indices[i] = index;
	}
}

__global__ __launch_bounds__( 256 )
void spreadValuesKernel( const float* source, float* target, const int* indices, int index, int n )
{
	const int i = blockIdx.x * 256 + threadIdx.x;
	if( i < n && indices[i] == index ) {
		target[i] = source[i];
	}
}

// sums over the middle one of three dimensions: first is [following][dimension][preceding] ( :146-207 )
template<typename T, bool CUMULATIVE>
__global__ __launch_bounds__( 256 )
void sumAlongDimensionKernel( const T* first, T* result, int preceding, int dimension, int following, int reverse )
{
	const long long lines = static_cast<long long>( preceding ) * following;
	for( long long line = blockIdx.x * 256LL + threadIdx.x; line < lines; line += static_cast<long long>( gridDim.x ) * 256 ) {
		const long long f = line / preceding;
		const int p = static_cast<int>( line - f * preceding );
		const T* in = first + f * dimension * preceding + p;
		T sum = T();
		if( CUMULATIVE ) {
			T* out = result + f * dimension * preceding + p;
			for( int d = 0; d < dimension; ++d ) {
				const int at = reverse ? dimension - 1 - d : d;
				sum = d == 0 ? in[static_cast<long long>( at ) * preceding] : in[static_cast<long long>( at ) * preceding] + sum;
				out[static_cast<long long>( at ) * preceding] = sum;
			}
		} else {
			for( int d = 0; d < dimension; ++d ) {
				sum = d == 0 ? in[0] : in[static_cast<long long>( d ) * preceding] + sum;
			}
			result[line] = sum;
		}
	}
}

// The Jacobians of the two sums above as dense matrices ( :209-264 ): row ( f, p [, d] ), column ( f, k, p ) holds
// first[f][k][p] for every k ( for k <= d in the cumulative form ), zero elsewhere.
template<bool CUMULATIVE>
__global__ __launch_bounds__( 256 )
void sumAlongDimensionDiagKernel( const float* first, float* result, int preceding, int dimension, int following, long long total )
{
	const long long width = static_cast<long long>( preceding ) * dimension * following;
	for( long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += static_cast<long long>( gridDim.x ) * 256 ) {
		const long long row = i / width;
		const long long column = i - row * width;
		// row = ( f * preceding + p ) [ * dimension + d ]
		const long long fp = CUMULATIVE ? row / dimension : row;
		const int d = CUMULATIVE ? static_cast<int>( row - fp * dimension ) : dimension - 1;
		const long long f = fp / preceding;
		const int p = static_cast<int>( fp - f * preceding );
		const long long cf = column / ( static_cast<long long>( dimension ) * preceding );
		const long long rest = column - cf * dimension * preceding;
		const int k = static_cast<int>( rest / preceding );
		const int cp = static_cast<int>( rest - static_cast<long long>( k ) * preceding );
		result[i] = ( cf == f && cp == p && k <= d ) ? first[( f * dimension + k ) * preceding + p] : 0.f;
	}
}

} // namespace nh

extern "C" int nhFilterSmallValues( nhStream s, float* data, int dataSize, float threshold )
{
	CFilterSmallOp op; op.Threshold = threshold;
	return launchEltwise<1, float, float>( s, data, (const float*)nullptr, (const float*)nullptr, data, dataSize, op );
}
extern "C" int nhVectorSumAdd( nhStream s, const float* first, int vectorSize, float* result )
{
	NH_REQUIRE( vectorSize >= 0 && result != nullptr );
	return launchSum<false>( s, first, nullptr, vectorSize, result, true );
}
extern "C" int nhVectorEqualInt( nhStream s, const int* first, const int* second, float* result, int vectorSize )
{
	return launchEltwise<2, int, float>( s, first, second, (const int*)nullptr, result, vectorSize, CEqualToFloatOp() );
}
extern "C" int nhVectorEqualValueInt( nhStream s, const int* first, float* result, int vectorSize, const int* value )
{
	NH_REQUIRE( value != nullptr );
	CEqualValueOp op; op.Ptr = value; op.Value = 0;
	return launchEltwise<1, int, float>( s, first, (const int*)nullptr, (const int*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMax( nhStream s, const float* first, float secondValue, float* result, int vectorSize )
{
	CMaxValueOp op; op.Value = secondValue;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorMaxDiff( nhStream s, const float* first, float secondValue, float* grad, int gradHeight, int gradWidth )
{
	CRowMaxDiff f; f.Value = secondValue;
	return launchRowCondition( s, first, grad, grad, gradHeight, gradWidth, f );
}
extern "C" int nhVectorAbsDiffRows( nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* first, float* result )
{
	return launchRowCondition( s, first, sourceGrad, result, gradHeight, gradWidth, CRowAbsDiff() );
}
extern "C" int nhVectorLogDiff( nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* value, float* result )
{
	return launchRowCondition( s, value, sourceGrad, result, gradHeight, gradWidth, CRowLogDiff() );
}
extern "C" int nhVectorMinMaxDiff( nhStream s, const float* sourceGrad, int gradHeight, int gradWidth, const float* first, float* result,
	const float* minValue, const float* maxValue )
{
	NH_REQUIRE( minValue != nullptr && maxValue != nullptr );
	CRowMinMaxDiff f; f.MinPtr = minValue; f.MaxPtr = maxValue;
	return launchRowCondition( s, first, sourceGrad, result, gradHeight, gradWidth, f );
}
extern "C" int nhVectorBernulliKLDerivative( nhStream s, const float* estimation, float* result, int vectorSize, const float* target )
{
	NH_REQUIRE( target != nullptr );
	CBernulliKLOp op; op.Ptr = target; op.Target = 0;
	return launchEltwise<1, float, float>( s, estimation, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
NH_BINARY( nhVectorEltwiseDivideInt, int, CDivIntOp )
NH_BINARY( nhVectorEltwisePower, float, CEltwisePowerOp )
extern "C" int nhVectorPower( nhStream s, float exponent, const float* first, float* result, int vectorSize )
{
	CPowerOp op; op.Exponent = exponent;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorPowerDiff( nhStream s, float exponent, const float* first, const float* second, float* result, int vectorSize )
{
	CPowerDiffOp op; op.Exponent = exponent; op.Power = exponent - 1.f;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorPowerDiffOp( nhStream s, float exponent, const float* first, const float* second, float* result, int vectorSize )
{
	CPowerDiffOp op; op.Exponent = exponent; op.Power = ( exponent - 1.f ) / exponent;
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorEltwiseNotInt( nhStream s, const int* first, int* result, int vectorSize )
{
	return launchEltwise<1, int, int>( s, first, (const int*)nullptr, (const int*)nullptr, result, vectorSize, CNotOp() );
}
extern "C" int nhVectorEltwiseNotNegative( nhStream s, const int* first, float* result, int vectorSize )
{
	return launchEltwise<1, int, float>( s, first, (const int*)nullptr, (const int*)nullptr, result, vectorSize, CNotNegativeOp() );
}
extern "C" int nhVectorEltwiseLess( nhStream s, const float* first, const float* second, float* result, int vectorSize )
{
	return launchEltwise<2, float, float>( s, first, second, (const float*)nullptr, result, vectorSize, CLessOp<float, float>() );
}
extern "C" int nhVectorEltwiseLessValue( nhStream s, const float* first, float second, float* result, int vectorSize, int valueFirst )
{
	CLessValueOp op; op.Value = second; op.Reverse = valueFirst;
	return launchEltwise<1, float, float>( s, first, (const float*)nullptr, (const float*)nullptr, result, vectorSize, op );
}
extern "C" int nhVectorEltwiseLessToInt( nhStream s, const float* first, const float* second, int* result, int vectorSize )
{
	return launchEltwise<2, float, int>( s, first, second, (const float*)nullptr, result, vectorSize, CLessOp<float, int>() );
}
extern "C" int nhVectorEltwiseLessInt( nhStream s, const int* first, const int* second, int* result, int vectorSize )
{
	return launchEltwise<2, int, int>( s, first, second, (const int*)nullptr, result, vectorSize, CLessOp<int, int>() );
}
extern "C" int nhVectorEltwiseEqualToInt( nhStream s, const float* first, const float* second, int* result, int vectorSize )
{
	return launchEltwise<2, float, int>( s, first, second, (const float*)nullptr, result, vectorSize, CEqualToIntOp<float>() );
}
extern "C" int nhVectorEltwiseEqualInt( nhStream s, const int* first, const int* second, int* result, int vectorSize )
{
	return launchEltwise<2, int, int>( s, first, second, (const int*)nullptr, result, vectorSize, CEqualToIntOp<int>() );
}
extern "C" int nhVectorEltwiseWhere( nhStream s, const int* first, const void* second, const void* third, void* result, int vectorSize )
{
	return launchEltwise<3, int, int>( s, first, static_cast<const int*>( second ), static_cast<const int*>( third ),
		static_cast<int*>( result ), vectorSize, CWhereOp() );
}
extern "C" int nhVectorMaxWithIndex( nhStream s, const float* candidate, float* result, int* indices, int index, int vectorSize )
{
	NH_REQUIRE( vectorSize >= 0 );
	if( vectorSize == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( candidate != nullptr && result != nullptr && indices != nullptr );
	hipLaunchKernelGGL( maxWithIndexKernel, dim3( ceilDiv( vectorSize, 256 ) ), dim3( 256 ), 0, toStream( s ), candidate, result, indices,
		index, vectorSize );
	NH_LAUNCH_CHECK();
	return NH_OK;
}
extern "C" int nhVectorSpreadValuesTo( nhStream s, const float* source, float* target, const int* indices, int index, int vectorSize )
{
	NH_REQUIRE( vectorSize >= 0 );
	if( vectorSize == 0 ) {
		return NH_OK;
	}
	NH_REQUIRE( source != nullptr && target != nullptr && indices != nullptr );
	hipLaunchKernelGGL( spreadValuesKernel, dim3( ceilDiv( vectorSize, 256 ) ), dim3( 256 ), 0, toStream( s ), source, target, indices,
		index, vectorSize );
	NH_LAUNCH_CHECK();
	return NH_OK;
}

template<typename T, bool CUMULATIVE>
static int launchSumAlongDimension( nhStream s, const T* first, int preceding, int dimension, int following, T* result, int reverse )
{
	NH_REQUIRE( preceding > 0 && dimension > 0 && following > 0 && first != nullptr && result != nullptr );
	const long long lines = static_cast<long long>( preceding ) * following;
	const long long blocks = ( lines + 255 ) / 256;
	hipLaunchKernelGGL( ( sumAlongDimensionKernel<T, CUMULATIVE> ), dim3( static_cast<unsigned>( blocks > 8192 ? 8192 : blocks ) ), dim3( 256 ), 0,
		toStream( s ), first, result, preceding, dimension, following, reverse );
	NH_LAUNCH_CHECK();
	return NH_OK;
}
extern "C" int nhVectorSumAlongDimension( nhStream s, const float* first, int precedingDimension, int dimension, int followingDimension,
	float* result )
{
	return launchSumAlongDimension<float, false>( s, first, precedingDimension, dimension, followingDimension, result, 0 );
}
extern "C" int nhVectorCumSumAlongDimension( nhStream s, const float* first, int precedingDimension, int dimension, int followingDimension,
	float* result, int reverse )
{
	return launchSumAlongDimension<float, true>( s, first, precedingDimension, dimension, followingDimension, result, reverse );
}
extern "C" int nhVectorCumSumAlongDimensionInt( nhStream s, const int* first, int precedingDimension, int dimension, int followingDimension,
	int* result, int reverse )
{
	return launchSumAlongDimension<int, true>( s, first, precedingDimension, dimension, followingDimension, result, reverse );
}
extern "C" int nhVectorSumAlongDimensionDiag( nhStream s, const float* first, int precedingDimension, int dimension, int followingDimension,
	float* result, int cumulative )
{
	NH_REQUIRE( precedingDimension > 0 && dimension > 0 && followingDimension > 0 && first != nullptr && result != nullptr );
	const long long width = static_cast<long long>( precedingDimension ) * dimension * followingDimension;
	const long long rows = static_cast<long long>( precedingDimension ) * followingDimension * ( cumulative ? dimension : 1 );
	const long long total = width * rows;
	const long long blocks = ( total + 255 ) / 256;
	const dim3 grid( static_cast<unsigned>( blocks > 8192 ? 8192 : blocks ) );
	if( cumulative ) {
		hipLaunchKernelGGL( sumAlongDimensionDiagKernel<true>, grid, dim3( 256 ), 0, toStream( s ), first, result, precedingDimension, dimension,
			followingDimension, total );
	} else {
		hipLaunchKernelGGL( sumAlongDimensionDiagKernel<false>, grid, dim3( 256 ), 0, toStream( s ), first, result, precedingDimension, dimension,
			followingDimension, total );
	}
	NH_LAUNCH_CHECK();
	return NH_OK;
}
