// A small test framework that understands the subset of the Google Test vocabulary which NeoMathEngine's own
// test sources use ( TEST, TEST_F, TEST_P, INSTANTIATE_TEST_CASE_P, Values / ValuesIn, ASSERT_* / EXPECT_*,
// GTEST_LOG_, InitGoogleTest, RUN_ALL_TESTS, --gtest_filter, --gtest_list_tests ), so that those sources compile
// where they lie and run against any IMathEngine without the real library, which their build fetches from the network.
// Written for this purpose only: no death tests, matchers, typed tests, sharding or XML output.
#pragma once

// ( the real header brings these in, and the test sources count on it )
#include <cfloat>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <functional>
#include <initializer_list>
#include <iostream>
#include <limits>
#include <memory>
#include <sstream>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

namespace testing {

class Message {
public:
	Message() {}
	Message( const Message& other ) { text << other.text.str(); }
	template<class T> Message& operator<<( const T& value ) { text << value; return *this; }
	Message& operator<<( std::ostream& ( *manipulator )( std::ostream& ) ) { text << manipulator; return *this; }
	std::string str() const { return text.str(); }
private:
	std::ostringstream text;
};

namespace internal {

// What the running test has recorded so far.
struct CTestState {
	int Failures = 0;
	bool Fatal = false;
};
CTestState& CurrentTest();

class AssertHelper {
public:
	AssertHelper( const char* _file, int _line, bool _fatal, const std::string& _summary ) :
		file( _file ), line( _line ), fatal( _fatal ), summary( _summary ) {}
	void operator=( const Message& message ) const;
private:
	const char* file;
	int line;
	bool fatal;
	std::string summary;
};

template<class T, class = void> struct IsStreamable : std::false_type {};
template<class T> struct IsStreamable<T, decltype( void( std::declval<std::ostream&>() << std::declval<const T&>() ) )> : std::true_type {};

template<class T>
typename std::enable_if<IsStreamable<T>::value, std::string>::type Print( const T& value )
{
	std::ostringstream s;
	s.precision( 9 );
	s << value;
	return s.str();
}
template<class T>
typename std::enable_if<!IsStreamable<T>::value, std::string>::type Print( const T& )
{
	return "<value of " + std::to_string( sizeof( T ) ) + " bytes>";
}

template<class A, class B>
std::string CompareText( const char* op, const char* aText, const char* bText, const A& a, const B& b )
{
	return std::string( "Expected: (" ) + aText + ") " + op + " (" + bText + "), actual: " + Print( a ) + " vs " + Print( b );
}

// the comparison of the EXPECT_FLOAT_EQ family: within four units in the last place, NaN equals nothing
inline bool AlmostEqualFloats( float a, float b )
{
	if( std::isnan( a ) || std::isnan( b ) ) {
		return false;
	}
	auto biased = []( float f ) -> uint32_t {
		uint32_t bits;
		std::memcpy( &bits, &f, sizeof( bits ) );
		return ( bits & 0x80000000u ) != 0 ? ~bits + 1 : bits | 0x80000000u;
	};
	const uint32_t x = biased( a ), y = biased( b );
	return ( x > y ? x - y : y - x ) <= 4;
}

class LogLine {
public:
	explicit LogLine( const char* level, const char* file, int line ) { text << "[" << level << "] " << file << ":" << line << ": "; }
	~LogLine() { std::cerr << text.str() << std::endl; }
	std::ostream& stream() { return text; }
private:
	std::ostringstream text;
};

} // namespace internal

class Test {
public:
	virtual ~Test() {}
	virtual void SetUp() {}
	virtual void TearDown() {}
	virtual void TestBody() = 0;
	static bool HasFatalFailure() { return internal::CurrentTest().Fatal; }
	static bool HasFailure() { return internal::CurrentTest().Failures > 0; }
	static void SetUpTestCase() {}
	static void TearDownTestCase() {}
};

template<class T>
class WithParamInterface {
public:
	typedef T ParamType;
	virtual ~WithParamInterface() {}
	static const T& GetParam() { return *Current(); }
	static const T*& Current() { static const T* current = nullptr; return current; }
};

template<class T>
class TestWithParam : public Test, public WithParamInterface<T> {
};

// ---- parameter generators ------------------------------------------------------------------------------

namespace internal {

template<class... Ts>
class ValueList {
public:
	explicit ValueList( const Ts&... values ) : values_( values... ) {}
	template<class T> std::vector<T> As() const { std::vector<T> out; Append<T>( out, std::index_sequence_for<Ts...>() ); return out; }
private:
	template<class T, size_t... I> void Append( std::vector<T>& out, std::index_sequence<I...> ) const
	{
		( void )std::initializer_list<int>{ ( out.push_back( static_cast<T>( std::get<I>( values_ ) ) ), 0 )... };
	}
	std::tuple<Ts...> values_;
};

template<class V>
class ContainerValues {
public:
	explicit ContainerValues( std::vector<V> values ) : values_( std::move( values ) ) {}
	template<class T> std::vector<T> As() const { return std::vector<T>( values_.begin(), values_.end() ); }
private:
	std::vector<V> values_;
};

} // namespace internal

template<class... Ts>
internal::ValueList<Ts...> Values( const Ts&... values ) { return internal::ValueList<Ts...>( values... ); }

template<class Container>
auto ValuesIn( const Container& container ) -> internal::ContainerValues<typename std::decay<decltype( *std::begin( container ) )>::type>
{
	typedef typename std::decay<decltype( *std::begin( container ) )>::type V;
	return internal::ContainerValues<V>( std::vector<V>( std::begin( container ), std::end( container ) ) );
}

// ---- registry -------------------------------------------------------------------------------------------

namespace internal {

struct CTestCase {
	std::string Name;                  // "Suite.Test" or "Prefix/Suite.Test/Index"
	std::function<void()> Run;         // builds the fixture, binds the parameter, runs SetUp / TestBody / TearDown
};

// Suites with parameters keep their test bodies and their parameter sets apart until the tests are listed:
// a TEST_P and its INSTANTIATE_TEST_CASE_P may come in either order.
struct CParamSuite {
	virtual ~CParamSuite() {}
	virtual void Expand( std::vector<CTestCase>& out ) const = 0;
};

std::vector<CTestCase>& PlainTests();
std::vector<std::unique_ptr<CParamSuite>>& ParamSuites();
CParamSuite*& FindParamSuite( const std::string& name );
void RunOne( Test& test );

template<class Fixture>
class ParamSuiteOf : public CParamSuite {
public:
	typedef typename Fixture::ParamType P;
	static ParamSuiteOf& Get( const char* name )
	{
		CParamSuite*& slot = FindParamSuite( name );
		if( slot == nullptr ) {
			ParamSuiteOf* created = new ParamSuiteOf( name );
			ParamSuites().emplace_back( created );
			slot = created;
		}
		return *static_cast<ParamSuiteOf*>( slot );
	}
	int AddTest( const char* testName, std::function<Fixture*()> factory ) { tests.push_back( { testName, factory } ); return 0; }
	int AddParams( const char* prefix, std::vector<P> params ) { instantiations.push_back( { prefix, std::move( params ) } ); return 0; }

	void Expand( std::vector<CTestCase>& out ) const override
	{
		for( const auto& inst : instantiations ) {
			for( const auto& test : tests ) {
				for( size_t i = 0; i < inst.second.size(); ++i ) {
					const P* param = &inst.second[i];
					auto factory = test.second;
					out.push_back( { inst.first + "/" + suite + "." + test.first + "/" + std::to_string( i ), [param, factory]() {
						WithParamInterface<P>::Current() = param;
						std::unique_ptr<Fixture> fixture( factory() );
						RunOne( *fixture );
						WithParamInterface<P>::Current() = nullptr;
					} } );
				}
			}
		}
	}
private:
	explicit ParamSuiteOf( const char* name ) : suite( name ) {}
	std::string suite;
	std::vector<std::pair<std::string, std::function<Fixture*()>>> tests;
	std::vector<std::pair<std::string, std::vector<P>>> instantiations;
};

template<class TestClass>
int AddPlainTest( const char* suite, const char* name )
{
	PlainTests().push_back( { std::string( suite ) + "." + name, []() { TestClass test; RunOne( test ); } } );
	return 0;
}

} // namespace internal

void InitGoogleTest( int* argc, char** argv );
int RunAllTests();

} // namespace testing

#define RUN_ALL_TESTS() ::testing::RunAllTests()

// ---- test definitions -----------------------------------------------------------------------------------

#define GTEST_LITE_CLASS_( suite, name ) suite##_##name##_Test

#define GTEST_LITE_PLAIN_( suite, name, base ) \
	class GTEST_LITE_CLASS_( suite, name ) : public base { public: void TestBody() override; }; \
	static int gtest_lite_registered_##suite##_##name = ::testing::internal::AddPlainTest<GTEST_LITE_CLASS_( suite, name )>( #suite, #name ); \
	void GTEST_LITE_CLASS_( suite, name )::TestBody()

#define TEST( suite, name ) GTEST_LITE_PLAIN_( suite, name, ::testing::Test )
#define TEST_F( fixture, name ) GTEST_LITE_PLAIN_( fixture, name, fixture )

#define TEST_P( fixture, name ) \
	class GTEST_LITE_CLASS_( fixture, name ) : public fixture { public: void TestBody() override; }; \
	static int gtest_lite_registered_##fixture##_##name = ::testing::internal::ParamSuiteOf<fixture>::Get( #fixture ).AddTest( #name, \
		[]() -> fixture* { return new GTEST_LITE_CLASS_( fixture, name ); } ); \
	void GTEST_LITE_CLASS_( fixture, name )::TestBody()

#define INSTANTIATE_TEST_CASE_P( prefix, fixture, ... ) \
	static int gtest_lite_instantiated_##prefix##_##fixture = ::testing::internal::ParamSuiteOf<fixture>::Get( #fixture ).AddParams( #prefix, \
		( __VA_ARGS__ ).template As<fixture::ParamType>() )
#define INSTANTIATE_TEST_SUITE_P INSTANTIATE_TEST_CASE_P

// ---- assertions -----------------------------------------------------------------------------------------
// ( "switch( 0 ) case 0: default:" swallows the dangling else, "return helper = message" leaves a void function )

#define GTEST_LITE_CHECK_( ok, fatal, summary ) \
	switch( 0 ) case 0: default: \
		if( ok ) ; else \
			fatal ::testing::internal::AssertHelper( __FILE__, __LINE__, #fatal[0] == 'r', summary ) = ::testing::Message()

#define GTEST_LITE_BOOL_( cond, expected, fatal ) \
	GTEST_LITE_CHECK_( static_cast<bool>( cond ) == expected, fatal, std::string( "Value of: " #cond "\n  Expected: " ) + ( expected ? "true" : "false" ) )

#define GTEST_LITE_CMP_( a, b, op, fatal ) \
	GTEST_LITE_CHECK_( ( a ) op ( b ), fatal, ::testing::internal::CompareText( #op, #a, #b, ( a ), ( b ) ) )

#define GTEST_LITE_NEAR_( a, b, eps, fatal ) \
	GTEST_LITE_CHECK_( std::fabs( static_cast<double>( a ) - static_cast<double>( b ) ) <= static_cast<double>( eps ), fatal, \
		std::string( "The difference between " #a " and " #b " exceeds " #eps ": " ) + ::testing::internal::Print( a ) + " vs " + ::testing::internal::Print( b ) )

#define GTEST_LITE_FLOAT_EQ_( a, b, fatal ) \
	GTEST_LITE_CHECK_( ::testing::internal::AlmostEqualFloats( ( a ), ( b ) ), fatal, ::testing::internal::CompareText( "==", #a, #b, ( a ), ( b ) ) )

#define EXPECT_TRUE( cond ) GTEST_LITE_BOOL_( cond, true, )
#define EXPECT_FALSE( cond ) GTEST_LITE_BOOL_( cond, false, )
#define ASSERT_TRUE( cond ) GTEST_LITE_BOOL_( cond, true, return )
#define ASSERT_FALSE( cond ) GTEST_LITE_BOOL_( cond, false, return )

#define EXPECT_EQ( a, b ) GTEST_LITE_CMP_( a, b, ==, )
#define EXPECT_NE( a, b ) GTEST_LITE_CMP_( a, b, !=, )
#define EXPECT_LT( a, b ) GTEST_LITE_CMP_( a, b, <, )
#define EXPECT_LE( a, b ) GTEST_LITE_CMP_( a, b, <=, )
#define EXPECT_GT( a, b ) GTEST_LITE_CMP_( a, b, >, )
#define EXPECT_GE( a, b ) GTEST_LITE_CMP_( a, b, >=, )
#define ASSERT_EQ( a, b ) GTEST_LITE_CMP_( a, b, ==, return )
#define ASSERT_NE( a, b ) GTEST_LITE_CMP_( a, b, !=, return )
#define ASSERT_LT( a, b ) GTEST_LITE_CMP_( a, b, <, return )
#define ASSERT_LE( a, b ) GTEST_LITE_CMP_( a, b, <=, return )
#define ASSERT_GT( a, b ) GTEST_LITE_CMP_( a, b, >, return )
#define ASSERT_GE( a, b ) GTEST_LITE_CMP_( a, b, >=, return )

#define EXPECT_NEAR( a, b, eps ) GTEST_LITE_NEAR_( a, b, eps, )
#define ASSERT_NEAR( a, b, eps ) GTEST_LITE_NEAR_( a, b, eps, return )
#define EXPECT_FLOAT_EQ( a, b ) GTEST_LITE_FLOAT_EQ_( a, b, )
#define ASSERT_FLOAT_EQ( a, b ) GTEST_LITE_FLOAT_EQ_( a, b, return )

#define ADD_FAILURE() GTEST_LITE_CHECK_( false, , "Failed" )
#define FAIL() GTEST_LITE_CHECK_( false, return, "Failed" )
#define SUCCEED() GTEST_LITE_CHECK_( true, , "" )

#define GTEST_LOG_( level ) ::testing::internal::LogLine( #level, __FILE__, __LINE__ ).stream()
