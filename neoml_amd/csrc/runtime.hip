// Device, stream, raw memory, transfers and timing behind the C ABI.
#include "common.h"
#include <stdarg.h>
#include <string.h>

namespace nh {

static thread_local char lastError[512] = "";

void setLastError( const char* fmt, ... )
{
	va_list ap;
	va_start( ap, fmt );
	vsnprintf( lastError, sizeof( lastError ), fmt, ap );
	va_end( ap );
}

} // namespace nh

namespace nh {
// dnn_ops.hip
int checkSequenceGiveUps( hipStream_t stream );
void releaseSequenceStream( hipStream_t stream );
}

using namespace nh;

extern "C" {

const char* nhGetLastError( void )
{
	return lastError;
}

int nhGetDeviceCount( int* count )
{
	NH_REQUIRE( count != nullptr );
	*count = 0;
	const hipError_t err = hipGetDeviceCount( count );
	if( err != hipSuccess ) {
		// a machine without a GPU is not an error for enumeration
		( void )hipGetLastError();
		*count = 0;
	}
	return NH_OK;
}

int nhGetDeviceInfo( int device, char* name, size_t* totalMemory, size_t* freeMemory, int* computeUnits, int* waveSize )
{
	hipDeviceProp_t prop;
	NH_HIP( hipGetDeviceProperties( &prop, device ) );
	if( name != nullptr ) {
		snprintf( name, 256, "%s (%s)", prop.name, prop.gcnArchName );
	}
	if( computeUnits != nullptr ) {
		*computeUnits = prop.multiProcessorCount;
	}
	if( waveSize != nullptr ) {
		*waveSize = prop.warpSize;
	}
	if( totalMemory != nullptr || freeMemory != nullptr ) {
		int previous = 0;
		NH_HIP( hipGetDevice( &previous ) );
		NH_HIP( hipSetDevice( device ) );
		size_t freeBytes = 0, totalBytes = 0;
		NH_HIP( hipMemGetInfo( &freeBytes, &totalBytes ) );
		NH_HIP( hipSetDevice( previous ) );
		if( totalMemory != nullptr ) *totalMemory = totalBytes;
		if( freeMemory != nullptr ) *freeMemory = freeBytes;
	}
	return NH_OK;
}

int nhSetDevice( int device )
{
	NH_HIP( hipSetDevice( device ) );
	return NH_OK;
}

int nhStreamCreate( nhStream* stream )
{
	NH_REQUIRE( stream != nullptr );
	hipStream_t s = nullptr;
	NH_HIP( hipStreamCreate( &s ) ); // default priority
	*stream = s;
	return NH_OK;
}

int nhStreamDestroy( nhStream stream )
{
	if( stream != nullptr ) {
		// what the library keeps for the stream goes with it ( a later stream may be handed the same handle )
		NH_HIP( hipStreamSynchronize( toStream( stream ) ) );
		releaseSliceScratch( toStream( stream ), true );
		releaseSequenceStream( toStream( stream ) );
		releaseTinyQueue( toStream( stream ) );
		NH_HIP( hipStreamDestroy( toStream( stream ) ) );
	}
	return NH_OK;
}

int nhStreamSynchronize( nhStream stream )
{
	NH_HIP( hipStreamSynchronize( toStream( stream ) ) );
	return checkSequenceGiveUps( toStream( stream ) );
}

int nhRawAlloc( void** ptr, size_t size )
{
	NH_REQUIRE( ptr != nullptr );
	*ptr = nullptr;
	const hipError_t err = hipMalloc( ptr, size );
	if( err == hipErrorOutOfMemory ) {
		( void )hipGetLastError();
		setLastError( "nhRawAlloc: out of device memory (%zu bytes)", size );
		return NH_ERR_MEMORY;
	}
	NH_HIP( err );
	return NH_OK;
}

int nhRawFree( void* ptr )
{
	if( ptr != nullptr ) {
		flushAllTinyOps(); // a call that has been put aside may still name this block
		NH_HIP( hipFree( ptr ) );
	}
	return NH_OK;
}

int nhCopyHostToDevice( nhStream stream, void* dst, const void* src, size_t size )
{
	if( size == 0 ) return NH_OK;
	NH_REQUIRE( dst != nullptr && src != nullptr );
	NH_HIP( hipMemcpyAsync( dst, src, size, hipMemcpyHostToDevice, toStream( stream ) ) );
	NH_HIP( hipStreamSynchronize( toStream( stream ) ) );
	return NH_OK;
}

int nhCopyDeviceToHost( nhStream stream, void* dst, const void* src, size_t size )
{
	if( size == 0 ) return NH_OK;
	NH_REQUIRE( dst != nullptr && src != nullptr );
	NH_HIP( hipMemcpyAsync( dst, src, size, hipMemcpyDeviceToHost, toStream( stream ) ) );
	NH_HIP( hipStreamSynchronize( toStream( stream ) ) );
	return checkSequenceGiveUps( toStream( stream ) );
}

int nhCopyDeviceToDevice( nhStream stream, void* dst, const void* src, size_t size )
{
	if( size == 0 ) return NH_OK;
	NH_REQUIRE( dst != nullptr && src != nullptr );
	NH_HIP( hipMemcpyAsync( dst, src, size, hipMemcpyDeviceToDevice, toStream( stream ) ) );
	return NH_OK;
}

int nhHostAlloc( void** ptr, size_t size )
{
	NH_REQUIRE( ptr != nullptr );
	*ptr = nullptr;
	const hipError_t err = hipHostMalloc( ptr, size, hipHostMallocDefault );
	if( err == hipErrorOutOfMemory ) {
		( void )hipGetLastError();
		setLastError( "nhHostAlloc: out of pinned host memory (%zu bytes)", size );
		return NH_ERR_MEMORY;
	}
	NH_HIP( err );
	return NH_OK;
}

int nhHostFree( void* ptr )
{
	if( ptr != nullptr ) {
		NH_HIP( hipHostFree( ptr ) );
	}
	return NH_OK;
}

int nhEventCreate( nhEvent* event )
{
	NH_REQUIRE( event != nullptr );
	hipEvent_t e = nullptr;
	NH_HIP( hipEventCreate( &e ) );
	*event = e;
	return NH_OK;
}

int nhEventDestroy( nhEvent event )
{
	if( event != nullptr ) {
		NH_HIP( hipEventDestroy( reinterpret_cast<hipEvent_t>( event ) ) );
	}
	return NH_OK;
}

int nhEventRecord( nhEvent event, nhStream stream )
{
	NH_REQUIRE( event != nullptr );
	NH_HIP( hipEventRecord( reinterpret_cast<hipEvent_t>( event ), toStream( stream ) ) );
	return NH_OK;
}

int nhEventSynchronize( nhEvent event )
{
	NH_REQUIRE( event != nullptr );
	NH_HIP( hipEventSynchronize( reinterpret_cast<hipEvent_t>( event ) ) );
	return NH_OK;
}

int nhEventElapsedMs( nhEvent start, nhEvent stop, float* ms )
{
	NH_REQUIRE( start != nullptr && stop != nullptr && ms != nullptr );
	NH_HIP( hipEventElapsedTime( ms, reinterpret_cast<hipEvent_t>( start ), reinterpret_cast<hipEvent_t>( stop ) ) );
	return NH_OK;
}

} // extern "C"
