// The engine side of NeoMathEngine's own test suite: the two functions its fixture header declares
// ( NeoMathEngine/test/src/common/TestFixture.h:31-33: RunTests, MathEngine ) and main().
// The reference's fixture picks the engine by --MathEngine= and can only name the engines its own factory builds
// ( NeoMathEngine/test/src/common/TestFixture.cpp:89-173 ); this one adds "hip": CreateHipMathEngine from
// libNeoMathEngineHip.so, found through --HipEngineLibrary=<path>, the NEOML_HIP_ENGINE_LIBRARY variable, or next to
// this repository's layout as seen from the executable ( ../../neoml_amd/lib ).
#include <TestFixture.h>

#include <dlfcn.h>
#include <libgen.h>
#include <unistd.h>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <string>

namespace NeoMLTest {

static IMathEngine* mathEngine = nullptr;

IMathEngine& MathEngine()
{
	return *mathEngine;
}

static const char* argValue( int argc, char* argv[], const char* flag )
{
	const size_t length = std::strlen( flag );
	for( int i = 1; i < argc; ++i ) {
		if( std::strncmp( argv[i], flag, length ) == 0 ) {
			return argv[i] + length;
		}
	}
	return nullptr;
}

static std::string defaultHipLibrary()
{
	char path[PATH_MAX] = {};
	const ssize_t length = readlink( "/proc/self/exe", path, sizeof( path ) - 1 );
	if( length <= 0 ) {
		return "libNeoMathEngineHip.so";
	}
	return std::string( dirname( path ) ) + "/../../neoml_amd/lib/libNeoMathEngineHip.so";
}

static IMathEngine* createHipMathEngine( int argc, char* argv[] )
{
	const char* fromFlag = argValue( argc, argv, "--HipEngineLibrary=" );
	const char* fromEnv = std::getenv( "NEOML_HIP_ENGINE_LIBRARY" );
	const std::string library = fromFlag != nullptr ? fromFlag : ( fromEnv != nullptr ? fromEnv : defaultHipLibrary() );
	void* handle = dlopen( library.c_str(), RTLD_NOW | RTLD_GLOBAL );
	if( handle == nullptr ) {
		GTEST_LOG_( ERROR ) << "cannot load " << library << ": " << dlerror();
		return nullptr;
	}
	typedef IMathEngine* ( *TCreate )( int device, size_t memoryLimit, int flags );
	TCreate create = reinterpret_cast<TCreate>( dlsym( handle, "CreateHipMathEngine" ) );
	if( create == nullptr ) {
		GTEST_LOG_( ERROR ) << library << " does not export CreateHipMathEngine";
		return nullptr;
	}
	return create( /*device*/0, /*memoryLimit*/0, /*flags*/0 );
}

int RunTests( int argc, char* argv[] )
{
	::testing::InitGoogleTest( &argc, argv );
	const char* engine = argValue( argc, argv, "--MathEngine=" );
	if( engine != nullptr && std::strcmp( engine, "hip" ) == 0 ) {
		mathEngine = createHipMathEngine( argc, argv );
	} else {
		if( engine == nullptr || std::strcmp( engine, "cpu" ) != 0 ) {
			GTEST_LOG_( WARNING ) << "Unknown type of MathEngine, taking the CPU one";
		}
		mathEngine = CreateCpuMathEngine( /*memoryLimit*/0u );
	}
	if( mathEngine == nullptr ) {
		GTEST_LOG_( INFO ) << "Can't create MathEngine!";
		return 1;
	}
	CMathEngineInfo info;
	mathEngine->GetMathEngineInfo( info );
	GTEST_LOG_( INFO ) << "Using MathEngine: " << info.Name << ", memory limit = " << info.AvailableMemory;
	const int result = RUN_ALL_TESTS();
	delete mathEngine;
	mathEngine = nullptr;
	return result;
}

} // namespace NeoMLTest

int main( int argc, char* argv[] )
{
	return NeoMLTest::RunTests( argc, argv );
}
