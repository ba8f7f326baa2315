// The run-time half of gtest/gtest.h: the registry of tests, the filter, the runner.
#include <gtest/gtest.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <exception>
#include <map>

namespace testing {
namespace internal {

CTestState& CurrentTest()
{
	static CTestState state;
	return state;
}

std::vector<CTestCase>& PlainTests()
{
	static std::vector<CTestCase> tests;
	return tests;
}

std::vector<std::unique_ptr<CParamSuite>>& ParamSuites()
{
	static std::vector<std::unique_ptr<CParamSuite>> suites;
	return suites;
}

CParamSuite*& FindParamSuite( const std::string& name )
{
	static std::map<std::string, CParamSuite*> byName;
	return byName[name];
}

void AssertHelper::operator=( const Message& message ) const
{
	CTestState& state = CurrentTest();
	++state.Failures;
	state.Fatal = state.Fatal || fatal;
	// a test that compares a million elements one by one would otherwise print a million lines
	if( state.Failures <= 5 ) {
		std::printf( "%s:%d: Failure\n%s\n", file, line, summary.c_str() );
		const std::string extra = message.str();
		if( !extra.empty() ) {
			std::printf( "%s\n", extra.c_str() );
		}
	} else if( state.Failures == 6 ) {
		std::printf( "( further failures of this test are counted, not printed )\n" );
	}
}

// An exception ends the test as a failure: an engine reports a violated assertion or a missing operation by throwing.
void RunOne( Test& test )
{
	try {
		test.SetUp();
		if( !Test::HasFatalFailure() ) {
			test.TestBody();
		}
		test.TearDown();
	} catch( const std::exception& e ) {
		AssertHelper( "exception", 0, true, std::string( "exception thrown in the test body: " ) + e.what() ) = Message();
	} catch( ... ) {
		AssertHelper( "exception", 0, true, "unknown exception thrown in the test body" ) = Message();
	}
}

static std::string filterText = "*";
static bool listOnly = false;

// '*' and '?' wildcards, as in --gtest_filter
static bool matches( const char* pattern, const char* name )
{
	if( *pattern == '\0' ) {
		return *name == '\0';
	}
	if( *pattern == '*' ) {
		return matches( pattern + 1, name ) || ( *name != '\0' && matches( pattern, name + 1 ) );
	}
	return *name != '\0' && ( *pattern == '?' || *pattern == *name ) && matches( pattern + 1, name + 1 );
}

static bool matchesAny( const std::string& patterns, const std::string& name )
{
	size_t begin = 0;
	while( begin <= patterns.size() ) {
		size_t end = patterns.find( ':', begin );
		if( end == std::string::npos ) {
			end = patterns.size();
		}
		if( end > begin && matches( patterns.substr( begin, end - begin ).c_str(), name.c_str() ) ) {
			return true;
		}
		begin = end + 1;
	}
	return false;
}

// positive patterns, then '-' and the negative ones
static bool selected( const std::string& name )
{
	const size_t dash = filterText.find( '-' );
	const std::string positive = dash == std::string::npos ? filterText : filterText.substr( 0, dash );
	const std::string negative = dash == std::string::npos ? std::string() : filterText.substr( dash + 1 );
	return ( positive.empty() || matchesAny( positive, name ) ) && !matchesAny( negative, name );
}

} // namespace internal

void InitGoogleTest( int* argc, char** argv )
{
	static const char filterFlag[] = "--gtest_filter=";
	for( int i = 1; i < *argc; ++i ) {
		if( std::strncmp( argv[i], filterFlag, sizeof( filterFlag ) - 1 ) == 0 ) {
			internal::filterText = argv[i] + sizeof( filterFlag ) - 1;
		} else if( std::strcmp( argv[i], "--gtest_list_tests" ) == 0 ) {
			internal::listOnly = true;
		}
	}
}

int RunAllTests()
{
	using namespace internal;
	std::vector<CTestCase> all = PlainTests();
	for( const auto& suite : ParamSuites() ) {
		suite->Expand( all );
	}
	std::vector<const CTestCase*> chosen;
	for( const auto& test : all ) {
		if( selected( test.Name ) ) {
			chosen.push_back( &test );
		}
	}
	if( listOnly ) {
		for( const CTestCase* test : chosen ) {
			std::printf( "%s\n", test->Name.c_str() );
		}
		return 0;
	}
	std::printf( "[==========] Running %zu tests of %zu.\n", chosen.size(), all.size() );
	std::vector<std::string> failed;
	const auto start = std::chrono::steady_clock::now();
	for( const CTestCase* test : chosen ) {
		std::printf( "[ RUN      ] %s\n", test->Name.c_str() );
		std::fflush( stdout );
		CurrentTest() = CTestState();
		const auto t0 = std::chrono::steady_clock::now();
		test->Run();
		const long long ms = std::chrono::duration_cast<std::chrono::milliseconds>( std::chrono::steady_clock::now() - t0 ).count();
		if( CurrentTest().Failures > 0 ) {
			failed.push_back( test->Name );
			std::printf( "[  FAILED  ] %s (%lld ms, %d failed checks)\n", test->Name.c_str(), ms, CurrentTest().Failures );
		} else {
			std::printf( "[       OK ] %s (%lld ms)\n", test->Name.c_str(), ms );
		}
		std::fflush( stdout );
	}
	const long long total = std::chrono::duration_cast<std::chrono::milliseconds>( std::chrono::steady_clock::now() - start ).count();
	std::printf( "[==========] %zu tests ran. (%lld ms total)\n", chosen.size(), total );
	std::printf( "[  PASSED  ] %zu tests.\n", chosen.size() - failed.size() );
	if( !failed.empty() ) {
		std::printf( "[  FAILED  ] %zu tests, listed below:\n", failed.size() );
		for( const auto& name : failed ) {
			std::printf( "[  FAILED  ] %s\n", name.c_str() );
		}
	}
	std::fflush( stdout );
	return failed.empty() ? 0 : 1;
}

} // namespace testing
