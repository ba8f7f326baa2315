// Caching allocator for engine blobs: size-class free lists per thread on top of a raw allocator, a memory
// limit, usage statistics and a per-thread LIFO stack carved from pool blocks.
//
// Behaviour restated from the reference's memory layer (src/MemoryPool.cpp:81-88,141-170,275-323,
// src/MathEngineStackAllocator.cpp:196-320, src/MemoryEngineMixin.cpp:99-183):
//   - 42 size classes from 256 B to 1 GiB (powers of two and, from 2 KiB up, the 1.5x steps between them);
//     a request is rounded up to its class; freed blocks go to the free list of the thread that owns them;
//   - requests above the thread's threshold (default 1 GiB), or with reuse switched off, go straight to the
//     raw allocator and straight back on free;
//   - the raw allocator may hold at most `memoryLimit` bytes (0 = unlimited); when a request fails the calling
//     thread's cached blocks are released and the request is tried once more, then NH_ERR_MEMORY;
//   - CleanUp releases the cached blocks and the empty stack of the calling thread only;
//   - the stack grows in 64 KiB quanta; while it is empty its single block is re-allocated to the high-water
//     mark, so a steady-state workload ends up with one block and no raw allocations.
// On a GPU every raw allocation synchronises the device, which is what the cache is there to avoid.
#include "../../include/neoml_hip.h"

#include <algorithm>
#include <map>
#include <mutex>
#include <stdlib.h>
#include <thread>
#include <unordered_map>
#include <vector>

namespace nh {
void setLastError( const char* fmt, ... );
}

namespace {

constexpr size_t StackQuantum = 64 * 1024;
constexpr size_t StackAlignment = 256; // keeps stack blobs eligible for 128-bit accesses

std::vector<size_t> makeSizeClasses()
{
	std::vector<size_t> sizes = { 256, 512, 1024 };
	for( size_t p = 2048; p < ( size_t( 1 ) << 30 ); p <<= 1 ) {
		sizes.push_back( p );
		sizes.push_back( p + p / 2 );
	}
	sizes.push_back( size_t( 1 ) << 30 );
	return sizes;
}

const std::vector<size_t>& sizeClasses()
{
	static const std::vector<size_t> classes = makeSizeClasses();
	return classes;
}

struct CUsedBlock {
	size_t Size;             // bytes taken from the raw allocator
	int Class;               // size class, -1 for a direct allocation
	std::thread::id Owner;   // thread whose free list gets the block back
};

struct CStackBlock {
	char* Base;
	size_t BlockSize;
	size_t Used;
};

struct CThreadState {
	bool Reuse;
	size_t Threshold;
	std::vector<std::vector<void*>> FreeLists; // one per size class
	// stack
	std::vector<CStackBlock> Stack; // back() is the current block
	size_t StackCurrent = 0;
	size_t StackHighWater = 0;
};

class CPool {
public:
	CPool( int kind, size_t limit ) :
		kind( kind ), limit( limit == 0 ? SIZE_MAX : limit ), allocated( 0 ), peak( 0 ), freeSize( this->limit ) {}
	~CPool();

	int HeapAlloc( size_t size, void** ptr );
	int HeapFree( void* ptr );
	int Transfer( void* ptr, size_t size );
	int StackAlloc( size_t size, void** ptr );
	int StackFree( void* ptr );
	void CleanUp();

	void SetReuse( bool enable ) { std::lock_guard<std::mutex> lock( mutex ); state().Reuse = enable; }
	bool GetReuse() { std::lock_guard<std::mutex> lock( mutex ); return state().Reuse; }
	void SetThreshold( size_t t ) { std::lock_guard<std::mutex> lock( mutex ); state().Threshold = t; }
	size_t GetThreshold() { std::lock_guard<std::mutex> lock( mutex ); return state().Threshold; }
	size_t Peak() { std::lock_guard<std::mutex> lock( mutex ); return peak; }
	void ResetPeak() { std::lock_guard<std::mutex> lock( mutex ); peak = allocated; }
	size_t Current() { std::lock_guard<std::mutex> lock( mutex ); return allocated; }
	size_t InPools();

private:
	const int kind;
	const size_t limit;
	size_t allocated; // bytes held from the raw allocator, cached blocks included
	size_t peak;
	size_t freeSize;
	std::mutex mutex;
	std::map<std::thread::id, CThreadState> threads;
	std::unordered_map<void*, CUsedBlock> used;

	CThreadState& state();
	void* rawAlloc( size_t size );
	void rawFree( void* ptr, size_t size );
	void* tryAlloc( size_t size, CThreadState& st );
	void* heapAllocLocked( size_t size );
	void heapFreeLocked( void* ptr );
	void releaseCached( CThreadState& st );
};

CThreadState& CPool::state()
{
	const std::thread::id id = std::this_thread::get_id();
	auto it = threads.find( id );
	if( it == threads.end() ) {
		CThreadState st;
		st.Reuse = true;
		st.Threshold = sizeClasses().back();
		st.FreeLists.resize( sizeClasses().size() );
		it = threads.emplace( id, std::move( st ) ).first;
	}
	return it->second;
}

void* CPool::rawAlloc( size_t size )
{
	if( size > limit || allocated > limit - size ) {
		return nullptr;
	}
	void* ptr = nullptr;
	if( kind == 0 ) {
		if( nhRawAlloc( &ptr, size ) != NH_OK ) {
			ptr = nullptr;
		}
	} else {
		ptr = aligned_alloc( 256, ( size + 255 ) / 256 * 256 );
	}
	if( ptr != nullptr ) {
		allocated += size;
		peak = std::max( peak, allocated );
	}
	return ptr;
}

void CPool::rawFree( void* ptr, size_t size )
{
	allocated -= size;
	if( kind == 0 ) {
		nhRawFree( ptr );
	} else {
		free( ptr );
	}
}

void* CPool::tryAlloc( size_t size, CThreadState& st )
{
	if( !st.Reuse || size > st.Threshold ) {
		void* ptr = rawAlloc( size );
		if( ptr != nullptr ) {
			used[ptr] = CUsedBlock{ size, -1, std::this_thread::get_id() };
			freeSize -= size;
		}
		return ptr;
	}
	const std::vector<size_t>& classes = sizeClasses();
	const int cls = static_cast<int>( std::lower_bound( classes.begin(), classes.end(), size ) - classes.begin() );
	void* ptr = nullptr;
	if( !st.FreeLists[cls].empty() ) {
		ptr = st.FreeLists[cls].back();
		st.FreeLists[cls].pop_back();
	} else {
		ptr = rawAlloc( classes[cls] );
		if( ptr == nullptr ) {
			return nullptr;
		}
	}
	used[ptr] = CUsedBlock{ classes[cls], cls, std::this_thread::get_id() };
	freeSize -= classes[cls];
	return ptr;
}

void CPool::releaseCached( CThreadState& st )
{
	const std::vector<size_t>& classes = sizeClasses();
	for( size_t cls = 0; cls < st.FreeLists.size(); ++cls ) {
		for( void* ptr : st.FreeLists[cls] ) {
			rawFree( ptr, classes[cls] );
		}
		st.FreeLists[cls].clear();
	}
}

void* CPool::heapAllocLocked( size_t size )
{
	CThreadState& st = state();
	void* ptr = tryAlloc( size, st );
	if( ptr == nullptr ) {
		releaseCached( st );
		ptr = tryAlloc( size, st );
	}
	return ptr;
}

void CPool::heapFreeLocked( void* ptr )
{
	auto it = used.find( ptr );
	const CUsedBlock block = it->second;
	used.erase( it );
	freeSize += block.Size;
	if( block.Class < 0 ) {
		rawFree( ptr, block.Size );
		return;
	}
	auto owner = threads.find( block.Owner );
	if( owner == threads.end() ) {
		rawFree( ptr, block.Size );
		return;
	}
	owner->second.FreeLists[block.Class].push_back( ptr );
}

int CPool::HeapAlloc( size_t size, void** ptr )
{
	std::lock_guard<std::mutex> lock( mutex );
	*ptr = heapAllocLocked( size == 0 ? 1 : size );
	if( *ptr == nullptr ) {
		nh::setLastError( "HeapAlloc: cannot allocate %zu bytes (in use %zu, limit %zu)", size, allocated, limit );
		return NH_ERR_MEMORY;
	}
	return NH_OK;
}

int CPool::HeapFree( void* ptr )
{
	std::lock_guard<std::mutex> lock( mutex );
	if( used.find( ptr ) == used.end() ) {
		nh::setLastError( "HeapFree: the pointer was not allocated by this pool" );
		return NH_ERR_ARGUMENT;
	}
	heapFreeLocked( ptr );
	return NH_OK;
}

int CPool::Transfer( void* ptr, size_t size )
{
	std::lock_guard<std::mutex> lock( mutex );
	auto it = used.find( ptr );
	if( it == used.end() ) {
		nh::setLastError( "TransferHandleToThisThread: the pointer was not allocated by this pool" );
		return NH_ERR_ARGUMENT;
	}
	CUsedBlock& block = it->second;
	if( block.Class >= 0 ) {
		if( size > block.Size ) {
			nh::setLastError( "TransferHandleToThisThread: size exceeds the block" );
			return NH_ERR_ARGUMENT;
		}
		CThreadState& st = state();
		if( st.Reuse ) {
			block.Owner = std::this_thread::get_id();
		} else {
			block.Class = -1; // leaves the caches: freed straight to the raw allocator
		}
	}
	return NH_OK;
}

int CPool::StackAlloc( size_t size, void** ptr )
{
	std::lock_guard<std::mutex> lock( mutex );
	size = ( std::max<size_t>( size, 1 ) + StackAlignment - 1 ) / StackAlignment * StackAlignment;
	CThreadState& st = state();
	st.StackCurrent += size;
	st.StackHighWater = std::max( st.StackHighWater, st.StackCurrent );

	const bool regrow = st.Stack.size() == 1 && st.Stack[0].Used == 0 && st.Stack[0].BlockSize < st.StackHighWater;
	if( st.Stack.empty() || regrow ) {
		if( regrow ) {
			heapFreeLocked( st.Stack[0].Base );
			st.Stack.clear();
		}
		const size_t blockSize = ( st.StackHighWater + StackQuantum - 1 ) / StackQuantum * StackQuantum;
		void* base = heapAllocLocked( blockSize );
		if( base == nullptr ) {
			st.StackCurrent -= size;
			nh::setLastError( "StackAlloc: cannot allocate a %zu byte stack block", blockSize );
			return NH_ERR_MEMORY;
		}
		st.Stack.push_back( CStackBlock{ static_cast<char*>( base ), blockSize, size } );
		*ptr = base;
		return NH_OK;
	}
	CStackBlock& top = st.Stack.back();
	if( top.Used + size <= top.BlockSize ) {
		*ptr = top.Base + top.Used;
		top.Used += size;
		return NH_OK;
	}
	const size_t blockSize = ( size + StackQuantum - 1 ) / StackQuantum * StackQuantum;
	void* base = heapAllocLocked( blockSize );
	if( base == nullptr ) {
		st.StackCurrent -= size;
		nh::setLastError( "StackAlloc: cannot allocate a %zu byte stack block", blockSize );
		return NH_ERR_MEMORY;
	}
	st.Stack.push_back( CStackBlock{ static_cast<char*>( base ), blockSize, size } );
	*ptr = base;
	return NH_OK;
}

int CPool::StackFree( void* ptr )
{
	if( ptr == nullptr ) {
		return NH_OK;
	}
	std::lock_guard<std::mutex> lock( mutex );
	CThreadState& st = state();
	if( st.Stack.empty() ) {
		nh::setLastError( "StackFree: the stack of this thread is empty" );
		return NH_ERR_ARGUMENT;
	}
	CStackBlock& top = st.Stack.back();
	char* p = static_cast<char*>( ptr );
	if( p < top.Base || p >= top.Base + top.Used ) {
		nh::setLastError( "StackFree: not the most recent stack allocation of this thread" );
		return NH_ERR_ARGUMENT;
	}
	const size_t offset = static_cast<size_t>( p - top.Base );
	st.StackCurrent -= top.Used - offset;
	top.Used = offset;
	if( top.Used == 0 && st.Stack.size() > 1 ) {
		heapFreeLocked( top.Base );
		st.Stack.pop_back();
	}
	return NH_OK;
}

void CPool::CleanUp()
{
	std::lock_guard<std::mutex> lock( mutex );
	auto it = threads.find( std::this_thread::get_id() );
	if( it == threads.end() ) {
		return;
	}
	CThreadState& st = it->second;
	if( st.Stack.size() == 1 && st.Stack[0].Used == 0 ) {
		heapFreeLocked( st.Stack[0].Base );
		st.Stack.clear();
		st.StackCurrent = 0;
		st.StackHighWater = 0;
	}
	releaseCached( st );
}

size_t CPool::InPools()
{
	std::lock_guard<std::mutex> lock( mutex );
	auto it = threads.find( std::this_thread::get_id() );
	if( it == threads.end() ) {
		return 0;
	}
	size_t total = 0;
	for( size_t cls = 0; cls < it->second.FreeLists.size(); ++cls ) {
		total += it->second.FreeLists[cls].size() * sizeClasses()[cls];
	}
	return total;
}

CPool::~CPool()
{
	for( auto& t : threads ) {
		for( CStackBlock& b : t.second.Stack ) {
			auto it = used.find( b.Base );
			if( it != used.end() ) {
				rawFree( b.Base, it->second.Size );
				used.erase( it );
			}
		}
		releaseCached( t.second );
	}
	// blocks the caller never freed
	for( auto& u : used ) {
		rawFree( u.first, u.second.Size );
	}
}

} // namespace

#define NH_POOL_REQUIRE( expr ) \
	do { if( !( expr ) ) { nh::setLastError( "%s: requirement failed: %s", __func__, #expr ); return NH_ERR_ARGUMENT; } } while( 0 )

extern "C" {

int nhPoolCreate( nhPool* pool, int kind, size_t memoryLimit )
{
	NH_POOL_REQUIRE( pool != nullptr && ( kind == 0 || kind == 1 ) );
	*pool = new CPool( kind, memoryLimit );
	return NH_OK;
}

int nhPoolDestroy( nhPool pool )
{
	delete static_cast<CPool*>( pool );
	return NH_OK;
}

int nhPoolSetReuseMemoryMode( nhPool pool, int enable )
{
	NH_POOL_REQUIRE( pool != nullptr );
	static_cast<CPool*>( pool )->SetReuse( enable != 0 );
	return NH_OK;
}

int nhPoolGetReuseMemoryMode( nhPool pool, int* enabled )
{
	NH_POOL_REQUIRE( pool != nullptr && enabled != nullptr );
	*enabled = static_cast<CPool*>( pool )->GetReuse() ? 1 : 0;
	return NH_OK;
}

int nhPoolSetThreadBufferMemoryThreshold( nhPool pool, size_t t )
{
	NH_POOL_REQUIRE( pool != nullptr );
	static_cast<CPool*>( pool )->SetThreshold( t );
	return NH_OK;
}

int nhPoolGetThreadBufferMemoryThreshold( nhPool pool, size_t* t )
{
	NH_POOL_REQUIRE( pool != nullptr && t != nullptr );
	*t = static_cast<CPool*>( pool )->GetThreshold();
	return NH_OK;
}

int nhPoolHeapAlloc( nhPool pool, size_t size, void** ptr )
{
	NH_POOL_REQUIRE( pool != nullptr && ptr != nullptr );
	return static_cast<CPool*>( pool )->HeapAlloc( size, ptr );
}

int nhPoolHeapFree( nhPool pool, void* ptr )
{
	NH_POOL_REQUIRE( pool != nullptr && ptr != nullptr );
	return static_cast<CPool*>( pool )->HeapFree( ptr );
}

int nhPoolTransferToThisThread( nhPool pool, void* ptr, size_t size )
{
	NH_POOL_REQUIRE( pool != nullptr && ptr != nullptr );
	return static_cast<CPool*>( pool )->Transfer( ptr, size );
}

int nhPoolStackAlloc( nhPool pool, size_t size, void** ptr )
{
	NH_POOL_REQUIRE( pool != nullptr && ptr != nullptr );
	return static_cast<CPool*>( pool )->StackAlloc( size, ptr );
}

int nhPoolStackFree( nhPool pool, void* ptr )
{
	NH_POOL_REQUIRE( pool != nullptr );
	return static_cast<CPool*>( pool )->StackFree( ptr );
}

int nhPoolCleanUp( nhPool pool )
{
	NH_POOL_REQUIRE( pool != nullptr );
	static_cast<CPool*>( pool )->CleanUp();
	return NH_OK;
}

int nhPoolGetPeakMemoryUsage( nhPool pool, size_t* bytes )
{
	NH_POOL_REQUIRE( pool != nullptr && bytes != nullptr );
	*bytes = static_cast<CPool*>( pool )->Peak();
	return NH_OK;
}

int nhPoolResetPeakMemoryUsage( nhPool pool )
{
	NH_POOL_REQUIRE( pool != nullptr );
	static_cast<CPool*>( pool )->ResetPeak();
	return NH_OK;
}

int nhPoolGetCurrentMemoryUsage( nhPool pool, size_t* bytes )
{
	NH_POOL_REQUIRE( pool != nullptr && bytes != nullptr );
	*bytes = static_cast<CPool*>( pool )->Current();
	return NH_OK;
}

int nhPoolGetMemoryInPools( nhPool pool, size_t* bytes )
{
	NH_POOL_REQUIRE( pool != nullptr && bytes != nullptr );
	*bytes = static_cast<CPool*>( pool )->InPools();
	return NH_OK;
}

} // extern "C"
