// engine_shim.cpp — drives a NeoML::IMathEngine through plain C calls on host buffers.
//
// TEST INFRASTRUCTURE ONLY. Compiled against the reference's public headers where they lie
// (/root/reference/NeoMathEngine/include) into oracle/_ref/; never linked into the shipped library.
// Every shim_* function takes an engine pointer, copies its host operands into blobs of that engine with
// DataExchangeRaw, calls exactly one interface method (the one the matching orc_* function of oracle.c restates)
// and copies the result back. With the engine returned by shim_create_cpu_engine() (the reference's own
// CCpuMathEngine, built from its sources by oracle/Makefile) this is the pin for the oracle and the
// "reference" CPU baseline; handed the HIP engine adapter, the same calls exercise the drop-in boundary.
#include <NeoMathEngine/NeoMathEngine.h>

#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

using namespace NeoML;

#define SHIM_API extern "C" __attribute__( ( visibility( "default" ) ) )

namespace {

thread_local std::string lastError;

// Blob of T on an engine, filled from / copied to host memory
template<class T>
class CBlob {
public:
	CBlob( IMathEngine& e, size_t size, const T* host = nullptr ) :
		engine( e ), size( size ), handle( e.HeapAllocTyped<T>( size == 0 ? 1 : size ) )
	{
		if( host != nullptr && size > 0 ) {
			engine.DataExchangeRaw( handle, host, size * sizeof( T ) );
		}
	}
	~CBlob() { engine.HeapFree( handle ); }
	CBlob( const CBlob& ) = delete;
	CBlob& operator=( const CBlob& ) = delete;

	const CTypedMemoryHandle<T>& Handle() const { return handle; }
	CTypedMemoryHandle<const T> Const() const { return handle; }
	void CopyTo( T* host ) const
	{
		if( size > 0 ) {
			engine.DataExchangeRaw( host, handle, size * sizeof( T ) );
		}
	}

private:
	IMathEngine& engine;
	size_t size;
	CTypedMemoryHandle<T> handle;
};

typedef CBlob<float> CFloatBlob;
typedef CBlob<int> CIntBlob;

CBlobDesc imageDesc( int n, int h, int w, int c )
{
	CBlobDesc d( CT_Float );
	d.SetDimSize( BD_BatchWidth, n );
	d.SetDimSize( BD_Height, h );
	d.SetDimSize( BD_Width, w );
	d.SetDimSize( BD_Channels, c );
	return d;
}

template<class F>
int guarded( F f )
{
	try {
		f();
		return 0;
	} catch( const std::bad_alloc& ) {
		lastError = "memory error";
		return 3;
	} catch( const std::exception& e ) {
		lastError = e.what();
		return 1;
	} catch( ... ) {
		lastError = "unknown exception";
		return 1;
	}
}

} // namespace

SHIM_API const char* shim_last_error() { return lastError.c_str(); }

SHIM_API void* shim_create_cpu_engine()
{
	try {
		return CreateCpuMathEngine( 0 );
	} catch( ... ) {
		return nullptr;
	}
}

SHIM_API void shim_destroy_engine( void* engine ) { delete static_cast<IMathEngine*>( engine ); }

SHIM_API int shim_engine_type( void* engine ) { return static_cast<IMathEngine*>( engine )->GetType(); }

// op codes as in oracle.c
enum {
	OP_RELU = 0, OP_ELU, OP_LEAKY_RELU, OP_HSWISH, OP_ABS, OP_HARD_TANH, OP_HARD_SIGMOID, OP_NEG,
	OP_EXP, OP_LOG, OP_ERF, OP_SQRT, OP_INV, OP_MINMAX, OP_SIGMOID, OP_TANH,
	OP_ADD_VALUE, OP_MULTIPLY, OP_NEG_MULTIPLY, OP_COPY, OP_NEG_LOG, OP_SUB_VALUE, OP_VALUE_SUB,
	OP_HINGE, OP_SQUARED_HINGE, OP_HUBER, OP_HUBER_DERIVATIVE
};

SHIM_API int shim_vector_unary( void* engine, int op, const float* first, float* result, int n, float p0, float p1 )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, n, first ), out( e, n ), s0( e, 1, &p0 ), s1( e, 1, &p1 );
		switch( op ) {
			case OP_RELU: e.VectorReLU( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_ELU: e.VectorELU( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_LEAKY_RELU: e.VectorLeakyReLU( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_HSWISH: e.VectorHSwish( in.Const(), out.Handle(), n ); break;
			case OP_ABS: e.VectorAbs( in.Const(), out.Handle(), n ); break;
			case OP_HARD_TANH: e.VectorHardTanh( in.Const(), out.Handle(), n ); break;
			case OP_HARD_SIGMOID: e.VectorHardSigmoid( in.Const(), out.Handle(), n, s0.Const(), s1.Const() ); break;
			case OP_NEG: e.VectorNeg( in.Const(), out.Handle(), n ); break;
			case OP_EXP: e.VectorExp( in.Const(), out.Handle(), n ); break;
			case OP_LOG: e.VectorLog( in.Const(), out.Handle(), n ); break;
			case OP_ERF: e.VectorErf( in.Const(), out.Handle(), n ); break;
			case OP_SQRT: e.VectorSqrt( in.Const(), out.Handle(), n ); break;
			case OP_INV: e.VectorInv( in.Const(), out.Handle(), n ); break;
			case OP_MINMAX: e.VectorMinMax( in.Const(), out.Handle(), n, s0.Const(), s1.Const() ); break;
			case OP_SIGMOID: e.VectorSigmoid( in.Const(), out.Handle(), n ); break;
			case OP_TANH: e.VectorTanh( in.Const(), out.Handle(), n ); break;
			case OP_ADD_VALUE: e.VectorAddValue( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_MULTIPLY: e.VectorMultiply( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_NEG_MULTIPLY: e.VectorNegMultiply( in.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_COPY: e.VectorCopy( out.Handle(), in.Const(), n ); break;
			case OP_NEG_LOG: e.VectorNegLog( in.Const(), out.Handle(), n ); break;
			case OP_HINGE: e.VectorHinge( in.Const(), out.Handle(), n ); break;
			case OP_SQUARED_HINGE: e.VectorSquaredHinge( in.Const(), out.Handle(), n ); break;
			case OP_HUBER: e.VectorHuber( in.Const(), out.Handle(), n ); break;
			case OP_HUBER_DERIVATIVE: e.VectorHuberDerivative( in.Const(), out.Handle(), n ); break;
			case OP_SUB_VALUE: e.VectorSub( in.Const(), p0, out.Handle(), n ); break;
			case OP_VALUE_SUB: e.VectorSub( p0, in.Const(), out.Handle(), n ); break;
			default: throw std::logic_error( "bad unary op" );
		}
		out.CopyTo( result );
	} );
}

enum {
	OP_ADD = 0, OP_SUB, OP_ELTWISE_MULTIPLY, OP_ELTWISE_NEG_MULTIPLY, OP_ELTWISE_DIVIDE, OP_ELTWISE_MAX,
	OP_ELTWISE_MIN, OP_MULTIPLY_AND_ADD, OP_MULTIPLY_AND_SUB, OP_ELTWISE_MULTIPLY_ADD,
	OP_RELU_DIFF, OP_HSWISH_DIFF, OP_SIGMOID_DIFF, OP_SIGMOID_DIFF_OP, OP_TANH_DIFF, OP_TANH_DIFF_OP,
	OP_ELU_DIFF, OP_ELU_DIFF_OP, OP_LEAKY_RELU_DIFF, OP_HARD_TANH_DIFF, OP_HARD_SIGMOID_DIFF, OP_HARD_SIGMOID_DIFF_OP,
	OP_ABS_DIFF, OP_HINGE_DIFF, OP_SQUARED_HINGE_DIFF, OP_L1_DIFF_ADD
};

SHIM_API int shim_vector_binary( void* engine, int op, const float* first, const float* second, float* result, int n, float p0,
	float p1 )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob a( e, n, first ), b( e, n, second ), out( e, n, result ), s0( e, 1, &p0 ), s1( e, 1, &p1 );
		switch( op ) {
			case OP_ADD: e.VectorAdd( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_SUB: e.VectorSub( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELTWISE_MULTIPLY: e.VectorEltwiseMultiply( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELTWISE_NEG_MULTIPLY: e.VectorEltwiseNegMultiply( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELTWISE_DIVIDE: e.VectorEltwiseDivide( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELTWISE_MAX: e.VectorEltwiseMax( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELTWISE_MIN: e.VectorEltwiseMin( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_MULTIPLY_AND_ADD: e.VectorMultiplyAndAdd( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_MULTIPLY_AND_SUB: e.VectorMultiplyAndSub( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_ELTWISE_MULTIPLY_ADD: e.VectorEltwiseMultiplyAdd( a.Const(), b.Const(), out.Handle(), n ); break;
			// both forms of the ReLU derivative are checked against each other: the second through the ReLU's output
			case OP_RELU_DIFF: e.VectorReLUDiff( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_HSWISH_DIFF: e.VectorHSwishDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_SIGMOID_DIFF: e.VectorSigmoidDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_SIGMOID_DIFF_OP: e.VectorSigmoidDiffOp( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_TANH_DIFF: e.VectorTanhDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_TANH_DIFF_OP: e.VectorTanhDiffOp( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_ELU_DIFF: e.VectorELUDiff( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_ELU_DIFF_OP: e.VectorELUDiffOp( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_LEAKY_RELU_DIFF: e.VectorLeakyReLUDiff( a.Const(), b.Const(), out.Handle(), n, s0.Const() ); break;
			case OP_HARD_TANH_DIFF: e.VectorHardTanhDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_HARD_SIGMOID_DIFF: e.VectorHardSigmoidDiff( a.Const(), b.Const(), out.Handle(), n, s0.Const(), s1.Const() ); break;
			case OP_HARD_SIGMOID_DIFF_OP: e.VectorHardSigmoidDiffOp( a.Const(), b.Const(), out.Handle(), n, s0.Const(), s1.Const() ); break;
			case OP_ABS_DIFF: e.VectorAbsDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_HINGE_DIFF: e.VectorHingeDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_SQUARED_HINGE_DIFF: e.VectorSquaredHingeDiff( a.Const(), b.Const(), out.Handle(), n ); break;
			case OP_L1_DIFF_ADD: e.VectorL1DiffAdd( a.Const(), b.Const(), out.Handle(), n, s0.Const(), s1.Const() ); break;
			default: throw std::logic_error( "bad binary op" );
		}
		out.CopyTo( result );
	} );
}

SHIM_API int shim_vector_binary_int( void* engine, int op, const int* first, const int* second, int* result, int n )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CIntBlob a( e, n, first ), b( e, n, second ), out( e, n );
		switch( op ) {
			case 0: e.VectorAdd( a.Const(), b.Const(), out.Handle(), n ); break;
			case 1: e.VectorSub( a.Const(), b.Const(), out.Handle(), n ); break;
			default: e.VectorEltwiseMultiply( a.Const(), b.Const(), out.Handle(), n ); break;
		}
		out.CopyTo( result );
	} );
}

SHIM_API int shim_vector_convert_float_to_int( void* engine, const float* from, int* to, int n )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, n, from );
		CIntBlob out( e, n );
		e.VectorConvert( in.Const(), out.Handle(), n );
		out.CopyTo( to );
	} );
}

SHIM_API int shim_vector_convert_int_to_float( void* engine, const int* from, float* to, int n )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CIntBlob in( e, n, from );
		CFloatBlob out( e, n );
		e.VectorConvert( in.Const(), out.Handle(), n );
		out.CopyTo( to );
	} );
}

SHIM_API int shim_vector_sum( void* engine, const float* first, int n, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, n, first ), out( e, 1 );
		e.VectorSum( in.Const(), n, out.Handle() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_vector_dot_product( void* engine, const float* first, const float* second, int n, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob a( e, n, first ), b( e, n, second ), out( e, 1 );
		e.VectorDotProduct( a.Const(), b.Const(), n, out.Handle() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_set_vector_to_matrix_rows( void* engine, float* result, int h, int w, const float* vec )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob v( e, w, vec ), out( e, size_t( h ) * w );
		e.SetVectorToMatrixRows( out.Handle(), h, w, v.Const() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_add_vector_to_matrix_rows( void* engine, int batch, const float* m, float* result, int h, int w, const float* vec )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const size_t n = size_t( batch ) * h * w;
		CFloatBlob in( e, n, m ), v( e, size_t( batch ) * w, vec ), out( e, n );
		e.AddVectorToMatrixRows( batch, in.Const(), out.Handle(), h, w, v.Const() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_add_vector_to_matrix_columns( void* engine, const float* m, float* result, int h, int w, const float* vec, int sign )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const size_t n = size_t( h ) * w;
		CFloatBlob in( e, n, m ), v( e, h, vec ), out( e, n );
		if( sign > 0 ) {
			e.AddVectorToMatrixColumns( in.Const(), out.Handle(), h, w, v.Const() );
		} else {
			e.SubVectorFromMatrixColumns( in.Const(), out.Handle(), h, w, v.Const() );
		}
		out.CopyTo( result );
	} );
}

SHIM_API int shim_sum_matrix_rows( void* engine, int batch, float* result, const float* m, int h, int w, int add )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( batch ) * h * w, m ), out( e, size_t( batch ) * w, result );
		if( add ) {
			e.SumMatrixRowsAdd( batch, out.Handle(), in.Const(), h, w );
		} else {
			e.SumMatrixRows( batch, out.Handle(), in.Const(), h, w );
		}
		out.CopyTo( result );
	} );
}

SHIM_API int shim_sum_matrix_columns( void* engine, float* result, const float* m, int h, int w )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( h ) * w, m ), out( e, h );
		e.SumMatrixColumns( out.Handle(), in.Const(), h, w );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_multiply_diag_matrix_by_matrix( void* engine, const float* diag, int n, const float* m, int w, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob d( e, n, diag ), in( e, size_t( n ) * w, m ), out( e, size_t( n ) * w );
		e.MultiplyDiagMatrixByMatrix( d.Const(), n, in.Const(), w, out.Handle(), n * w );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_batch_multiply_matrix_by_diag_matrix( void* engine, int batch, const float* first, int h, int w,
	int firstOffset, const float* second, int secondOffset, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const size_t firstSize = size_t( batch - 1 ) * firstOffset + size_t( h ) * w;
		const size_t secondSize = size_t( batch - 1 ) * secondOffset + w;
		CFloatBlob a( e, firstSize, first ), b( e, secondSize, second ), out( e, size_t( batch ) * h * w );
		e.BatchMultiplyMatrixByDiagMatrix( batch, a.Const(), h, w, firstOffset, b.Const(), secondOffset, out.Handle(), batch * h * w );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_matrix_softmax_by_rows( void* engine, const float* m, int h, int w, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( h ) * w, m ), out( e, size_t( h ) * w );
		e.MatrixSoftmaxByRows( in.Const(), h, w, out.Handle() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_matrix_log_sum_exp_by_rows( void* engine, const float* m, int h, int w, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( h ) * w, m ), out( e, h );
		e.MatrixLogSumExpByRows( in.Const(), h, w, out.Handle(), h );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_find_max_value_in_rows( void* engine, const float* m, int h, int w, float* result, int* indices )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( h ) * w, m ), out( e, h );
		CIntBlob idx( e, h );
		if( indices != nullptr ) {
			e.FindMaxValueInRows( in.Const(), h, w, out.Handle(), idx.Handle(), h );
			idx.CopyTo( indices );
		} else {
			e.FindMaxValueInRows( in.Const(), h, w, out.Handle(), h );
		}
		out.CopyTo( result );
	} );
}

SHIM_API int shim_find_max_value_in_columns( void* engine, int batch, const float* m, int h, int w, float* result, int* indices )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, size_t( batch ) * h * w, m ), out( e, size_t( batch ) * w );
		CIntBlob idx( e, size_t( batch ) * w );
		e.FindMaxValueInColumns( batch, in.Const(), h, w, out.Handle(), idx.Handle(), batch * w );
		out.CopyTo( result );
		idx.CopyTo( indices );
	} );
}

SHIM_API int shim_transpose_matrix( void* engine, int batch, const float* in, int h, int med, int w, int c, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const size_t n = size_t( batch ) * h * med * w * c;
		CFloatBlob a( e, n, in ), r( e, n );
		e.TransposeMatrix( batch, a.Const(), h, med, w, c, r.Handle(), static_cast<int>( n ) );
		r.CopyTo( out );
	} );
}

SHIM_API int shim_transpose_matrix_int( void* engine, int batch, const int* in, int h, int med, int w, int c, int* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const size_t n = size_t( batch ) * h * med * w * c;
		CIntBlob a( e, n, in ), r( e, n );
		e.TransposeMatrix( batch, a.Const(), h, med, w, c, r.Handle(), static_cast<int>( n ) );
		r.CopyTo( out );
	} );
}

// kind: 0 = A * B^T (strided), 1 = batched A * B^T, 2 = batched A * B, 3 = batched A^T * B, 4 = A^T * B added to C.
// Shapes in the orc_matmul_* convention: C is M x N, the reduction has length K.
SHIM_API int shim_matmul( void* engine, int kind, int batch, const float* a, int lda, const float* b, int ldb,
	float* c, int ldc, int M, int N, int K )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const bool aTransposed = kind == 3 || kind == 4;
		const bool bTransposed = kind == 0 || kind == 1;
		const size_t aRows = aTransposed ? K : M, bRows = bTransposed ? N : K;
		const size_t aSize = kind == 0 || kind == 4 ? ( aRows - 1 ) * lda + ( aTransposed ? M : K ) : size_t( batch ) * aRows * lda;
		const size_t bSize = kind == 0 || kind == 4 ? ( bRows - 1 ) * ldb + ( bTransposed ? K : N ) : size_t( batch ) * bRows * ldb;
		const size_t cSize = kind == 0 || kind == 4 ? size_t( M - 1 ) * ldc + N : size_t( batch ) * M * ldc;
		CFloatBlob A( e, aSize, a ), B( e, bSize, b ), C( e, cSize, c );
		switch( kind ) {
			case 0:
				e.MultiplyMatrixByTransposedMatrix( A.Const(), M, K, lda, B.Const(), N, ldb, C.Handle(), ldc, static_cast<int>( cSize ) );
				break;
			case 1:
				e.MultiplyMatrixByTransposedMatrix( batch, A.Const(), M, K, B.Const(), N, C.Handle(), static_cast<int>( cSize ) );
				break;
			case 2:
				e.MultiplyMatrixByMatrix( batch, A.Const(), M, K, B.Const(), N, C.Handle(), static_cast<int>( cSize ) );
				break;
			case 3:
				e.MultiplyTransposedMatrixByMatrix( batch, A.Const(), K, M, B.Const(), N, C.Handle(), static_cast<int>( cSize ) );
				break;
			case 4:
				e.MultiplyTransposedMatrixByMatrixAndAdd( A.Const(), K, M, lda, B.Const(), N, ldb, C.Handle(), ldc, static_cast<int>( cSize ) );
				break;
			default: throw std::logic_error( "bad matmul kind" );
		}
		C.CopyTo( c );
	} );
}

SHIM_API int shim_blob_convolution( void* engine, const float* in, int n, int h, int w, int cin, const float* filter,
	int cout, int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, const float* bias, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - ( fh - 1 ) * dh + 2 * ph - 1 ) / sh;
		const int wo = 1 + ( w - ( fw - 1 ) * dw + 2 * pw - 1 ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, cin ), filterDesc = imageDesc( cout, fh, fw, cin ),
			outDesc = imageDesc( n, ho, wo, cout );
		CFloatBlob src( e, inDesc.BlobSize(), in ), flt( e, filterDesc.BlobSize(), filter ), ft( e, cout, bias ),
			dst( e, outDesc.BlobSize() );
		CConvolutionDesc* desc = e.InitBlobConvolution( inDesc, ph, pw, sh, sw, dh, dw, filterDesc, outDesc );
		const CConstFloatHandle ftHandle = ft.Const();
		try {
			e.BlobConvolution( *desc, src.Const(), flt.Const(), bias != nullptr ? &ftHandle : nullptr, dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( out );
	} );
}

SHIM_API int shim_blob_channelwise_convolution( void* engine, const float* in, int n, int h, int w, int c,
	const float* filter, int fh, int fw, int ph, int pw, int sh, int sw, const float* bias, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - fh + 2 * ph ) / sh;
		const int wo = 1 + ( w - fw + 2 * pw ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), filterDesc = imageDesc( 1, fh, fw, c ),
			outDesc = imageDesc( n, ho, wo, c ), ftDesc = imageDesc( 1, 1, 1, c );
		CFloatBlob src( e, inDesc.BlobSize(), in ), flt( e, filterDesc.BlobSize(), filter ), ft( e, c, bias ),
			dst( e, outDesc.BlobSize() );
		CChannelwiseConvolutionDesc* desc = e.InitBlobChannelwiseConvolution( inDesc, ph, pw, sh, sw, filterDesc,
			bias != nullptr ? &ftDesc : nullptr, outDesc );
		const CConstFloatHandle ftHandle = ft.Const();
		try {
			e.BlobChannelwiseConvolution( *desc, src.Const(), flt.Const(), bias != nullptr ? &ftHandle : nullptr, dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( out );
	} );
}

// gradients of the channelwise convolution (NeoMathEngine.h:774-780); filterDiff and freeTermDiff (may be null) are
// accumulated into
SHIM_API int shim_blob_channelwise_convolution_backward( void* engine, const float* outDiff, int n, int h, int w, int c,
	const float* filter, int fh, int fw, int ph, int pw, int sh, int sw, float* inDiff )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - fh + 2 * ph ) / sh;
		const int wo = 1 + ( w - fw + 2 * pw ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), filterDesc = imageDesc( 1, fh, fw, c ),
			outDesc = imageDesc( n, ho, wo, c );
		CFloatBlob grad( e, outDesc.BlobSize(), outDiff ), flt( e, filterDesc.BlobSize(), filter ), dst( e, inDesc.BlobSize() );
		CChannelwiseConvolutionDesc* desc = e.InitBlobChannelwiseConvolution( inDesc, ph, pw, sh, sw, filterDesc, nullptr, outDesc );
		try {
			e.BlobChannelwiseConvolutionBackward( *desc, grad.Const(), flt.Const(), dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( inDiff );
	} );
}

SHIM_API int shim_blob_channelwise_convolution_learn_add( void* engine, const float* in, int n, int h, int w, int c,
	const float* outDiff, int fh, int fw, int ph, int pw, int sh, int sw, float* filterDiff, float* freeTermDiff )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - fh + 2 * ph ) / sh;
		const int wo = 1 + ( w - fw + 2 * pw ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), filterDesc = imageDesc( 1, fh, fw, c ),
			outDesc = imageDesc( n, ho, wo, c ), ftDesc = imageDesc( 1, 1, 1, c );
		CFloatBlob src( e, inDesc.BlobSize(), in ), grad( e, outDesc.BlobSize(), outDiff ),
			fd( e, filterDesc.BlobSize(), filterDiff ), ftd( e, c, freeTermDiff );
		CChannelwiseConvolutionDesc* desc = e.InitBlobChannelwiseConvolution( inDesc, ph, pw, sh, sw, filterDesc,
			freeTermDiff != nullptr ? &ftDesc : nullptr, outDesc );
		const CFloatHandle ftdHandle = ftd.Handle();
		try {
			e.BlobChannelwiseConvolutionLearnAdd( *desc, src.Const(), grad.Const(), fd.Handle(),
				freeTermDiff != nullptr ? &ftdHandle : nullptr );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		fd.CopyTo( filterDiff );
		if( freeTermDiff != nullptr ) {
			ftd.CopyTo( freeTermDiff );
		}
	} );
}

// The two fused blocks of depthwise-separable networks through the interface calls their layers make
// (MobileNetV2BlockLayer.cpp:205-250, ChannelwiseWith1x1Layer.cpp:150-197). activation codes: 0 none (AF_Linear),
// 1 ReLU (param = upper threshold when > 0), 2 h-swish. withExpand: MobileNetV2Block, else ChannelwiseWith1x1
// (then inputChannels is not used and expandedChannels is the input's channel count).
// inPlace != 0 (residual blocks only): output blob = input blob, as CDnn does when it reuses memory.
SHIM_API int shim_separable_block( void* engine, int withExpand, const float* in, int n, int h, int w, int inputChannels,
	int expandedChannels, int outputChannels, int stride, int residual, int expandActivation, float expandParam,
	int channelwiseActivation, float channelwiseParam, const float* expandFilter, const float* expandFreeTerm,
	const float* channelwiseFilter, const float* channelwiseFreeTerm, const float* downFilter, const float* downFreeTerm,
	int inPlace, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		static const TActivationFunction types[3] = { AF_Linear, AF_ReLU, AF_HSwish };
		const int blockInput = withExpand ? inputChannels : expandedChannels;
		const int ho = ( h + stride - 1 ) / stride, wo = ( w + stride - 1 ) / stride;
		const CBlobDesc inDesc = imageDesc( n, h, w, blockInput ), outDesc = imageDesc( n, ho, wo, outputChannels ),
			chInDesc = imageDesc( n, h, w, expandedChannels ), chOutDesc = imageDesc( n, ho, wo, expandedChannels ),
			chFilterDesc = imageDesc( 1, 3, 3, expandedChannels ), chFreeTermDesc = imageDesc( 1, 1, 1, expandedChannels );
		if( inPlace && inDesc.BlobSize() != outDesc.BlobSize() ) {
			throw std::logic_error( "in-place block needs equal input and output sizes" );
		}
		CFloatBlob src( e, inDesc.BlobSize(), in ),
			dst( e, outDesc.BlobSize() ),
			exF( e, withExpand ? expandedChannels * inputChannels : 1, withExpand ? expandFilter : nullptr ),
			exT( e, expandedChannels, expandFreeTerm ), chF( e, 9 * expandedChannels, channelwiseFilter ),
			chT( e, expandedChannels, channelwiseFreeTerm ), dnF( e, outputChannels * expandedChannels, downFilter ),
			dnT( e, outputChannels, downFreeTerm );
		const CConstFloatHandle exTh = exT.Const(), chTh = chT.Const(), dnTh = dnT.Const();
		CChannelwiseConvolutionDesc* convDesc = e.InitBlobChannelwiseConvolution( chInDesc, 1, 1, stride, stride, chFilterDesc,
			channelwiseFreeTerm != nullptr ? &chFreeTermDesc : nullptr, chOutDesc );
		CRowwiseOperationDesc* rowwise = withExpand
			? e.InitRowwiseMobileNetV2( inputChannels, exF.Const(), expandFreeTerm != nullptr ? &exTh : nullptr, expandedChannels,
				types[expandActivation], expandParam, chF.Const(), channelwiseFreeTerm != nullptr ? &chTh : nullptr, stride,
				types[channelwiseActivation], channelwiseParam, dnF.Const(), downFreeTerm != nullptr ? &dnTh : nullptr,
				outputChannels, residual != 0 )
			: e.InitRowwiseChWith1x1( stride, chF.Const(), channelwiseFreeTerm != nullptr ? &chTh : nullptr,
				types[channelwiseActivation], channelwiseParam, dnF.Const(), downFreeTerm != nullptr ? &dnTh : nullptr,
				outputChannels, residual != 0 );
		try {
			const CFloatHandle target = inPlace ? src.Handle() : dst.Handle();
			if( withExpand ) {
				e.MobileNetV2Block( inDesc, outDesc, *rowwise, *convDesc, src.Const(), target );
			} else {
				e.ChannelwiseWith1x1( inDesc, outDesc, *rowwise, *convDesc, src.Const(), target );
			}
		} catch( ... ) {
			delete rowwise;
			delete convDesc;
			throw;
		}
		delete rowwise;
		delete convDesc;
		if( inPlace ) {
			src.CopyTo( out );
		} else {
			dst.CopyTo( out );
		}
	} );
}

// The halves of a MobileNetV3 block around its squeeze-and-excite branch, as CMobileNetV3PreSEBlockLayer and
// CMobileNetV3PostSEBlockLayer call them (MobileNetV3BlockLayer.cpp:150-175, 245-265). The depthwise stage has a square
// filter of `filterSize` (3 or 5) with padding ( filterSize - 1 ) / 2. Activation codes as for shim_separable_block.
SHIM_API int shim_mobilenetv3_pre_se( void* engine, const float* in, int n, int h, int w, int inputChannels,
	int expandedChannels, int filterSize, int stride, int expandActivation, float expandParam, int channelwiseActivation,
	float channelwiseParam, const float* expandFilter, const float* expandFreeTerm, const float* channelwiseFilter,
	const float* channelwiseFreeTerm, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		static const TActivationFunction types[3] = { AF_Linear, AF_ReLU, AF_HSwish };
		const int pad = ( filterSize - 1 ) / 2;
		const int ho = ( h + 2 * pad - filterSize ) / stride + 1, wo = ( w + 2 * pad - filterSize ) / stride + 1;
		const CBlobDesc inDesc = imageDesc( n, h, w, inputChannels ), chInDesc = imageDesc( n, h, w, expandedChannels ),
			outDesc = imageDesc( n, ho, wo, expandedChannels ), chFilterDesc = imageDesc( 1, filterSize, filterSize, expandedChannels ),
			chFreeTermDesc = imageDesc( 1, 1, 1, expandedChannels );
		CFloatBlob src( e, inDesc.BlobSize(), in ), dst( e, outDesc.BlobSize() ),
			exF( e, expandedChannels * inputChannels, expandFilter ), exT( e, expandedChannels, expandFreeTerm ),
			chF( e, filterSize * filterSize * expandedChannels, channelwiseFilter ), chT( e, expandedChannels, channelwiseFreeTerm );
		const CConstFloatHandle exTh = exT.Const(), chTh = chT.Const();
		CChannelwiseConvolutionDesc* convDesc = e.InitBlobChannelwiseConvolution( chInDesc, pad, pad, stride, stride, chFilterDesc,
			channelwiseFreeTerm != nullptr ? &chFreeTermDesc : nullptr, outDesc );
		try {
			e.MobileNetV3PreSEBlock( inDesc, outDesc, *convDesc, src.Const(), exF.Const(),
				expandFreeTerm != nullptr ? &exTh : nullptr, types[expandActivation], expandParam, chF.Const(),
				channelwiseFreeTerm != nullptr ? &chTh : nullptr, types[channelwiseActivation], channelwiseParam, dst.Handle() );
		} catch( ... ) {
			delete convDesc;
			throw;
		}
		delete convDesc;
		dst.CopyTo( out );
	} );
}

SHIM_API int shim_mobilenetv3_post_se( void* engine, const float* in, int n, int h, int w, int channels, int outputChannels,
	const float* squeezeAndExcite, const float* residual, int activation, float param, const float* downFilter,
	const float* downFreeTerm, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		static const TActivationFunction types[3] = { AF_Linear, AF_ReLU, AF_HSwish };
		const CBlobDesc inDesc = imageDesc( n, h, w, channels ), outDesc = imageDesc( n, h, w, outputChannels );
		CFloatBlob src( e, inDesc.BlobSize(), in ), dst( e, outDesc.BlobSize() ), se( e, n * channels, squeezeAndExcite ),
			res( e, outDesc.BlobSize(), residual ), dnF( e, outputChannels * channels, downFilter ),
			dnT( e, outputChannels, downFreeTerm );
		const CConstFloatHandle resH = res.Const(), dnTh = dnT.Const();
		e.MobileNetV3PostSEBlock( inDesc, outputChannels, src.Const(), se.Const(), residual != nullptr ? &resH : nullptr,
			types[activation], param, dnF.Const(), downFreeTerm != nullptr ? &dnTh : nullptr, dst.Handle() );
		dst.CopyTo( out );
	} );
}

// gradients of the convolution through BlobConvolutionBackward / BlobConvolutionLearnAdd (NeoMathEngine.h:757-761);
// filterDiff and freeTermDiff (may be null) are accumulated into
SHIM_API int shim_blob_convolution_backward( void* engine, const float* outDiff, int n, int h, int w, int cin,
	const float* filter, int cout, int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, const float* bias,
	float* inDiff )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - ( fh - 1 ) * dh + 2 * ph - 1 ) / sh;
		const int wo = 1 + ( w - ( fw - 1 ) * dw + 2 * pw - 1 ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, cin ), filterDesc = imageDesc( cout, fh, fw, cin ),
			outDesc = imageDesc( n, ho, wo, cout );
		CFloatBlob src( e, outDesc.BlobSize(), outDiff ), flt( e, filterDesc.BlobSize(), filter ), ft( e, cin, bias ),
			dst( e, inDesc.BlobSize() );
		CConvolutionDesc* desc = e.InitBlobConvolution( inDesc, ph, pw, sh, sw, dh, dw, filterDesc, outDesc );
		const CConstFloatHandle ftHandle = ft.Const();
		try {
			e.BlobConvolutionBackward( *desc, src.Const(), flt.Const(), bias != nullptr ? &ftHandle : nullptr, dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( inDiff );
	} );
}

SHIM_API int shim_blob_convolution_learn_add( void* engine, const float* in, int n, int h, int w, int cin,
	const float* outDiff, int cout, int fh, int fw, int ph, int pw, int sh, int sw, int dh, int dw, float* filterDiff,
	float* freeTermDiff )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = 1 + ( h - ( fh - 1 ) * dh + 2 * ph - 1 ) / sh;
		const int wo = 1 + ( w - ( fw - 1 ) * dw + 2 * pw - 1 ) / sw;
		const CBlobDesc inDesc = imageDesc( n, h, w, cin ), filterDesc = imageDesc( cout, fh, fw, cin ),
			outDesc = imageDesc( n, ho, wo, cout );
		CFloatBlob src( e, inDesc.BlobSize(), in ), grad( e, outDesc.BlobSize(), outDiff ),
			fd( e, filterDesc.BlobSize(), filterDiff ), ftd( e, cout, freeTermDiff );
		CConvolutionDesc* desc = e.InitBlobConvolution( inDesc, ph, pw, sh, sw, dh, dw, filterDesc, outDesc );
		const CFloatHandle ftdHandle = ftd.Handle();
		try {
			e.BlobConvolutionLearnAdd( *desc, src.Const(), grad.Const(), fd.Handle(), freeTermDiff != nullptr ? &ftdHandle : nullptr, false );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		fd.CopyTo( filterDiff );
		if( freeTermDiff != nullptr ) {
			ftd.CopyTo( freeTermDiff );
		}
	} );
}

// forward max pooling with indices, then BlobMaxPoolingBackward with them (isMax) / BlobMeanPoolingBackward
SHIM_API int shim_blob_pooling_backward( void* engine, int isMax, const float* in, const float* resultDiff, int n, int h, int w,
	int c, int fh, int fw, int sh, int sw, float* sourceDiff )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = ( h - fh ) / sh + 1, wo = ( w - fw ) / sw + 1;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), outDesc = imageDesc( n, ho, wo, c );
		CFloatBlob src( e, inDesc.BlobSize(), in ), out( e, outDesc.BlobSize() ), grad( e, outDesc.BlobSize(), resultDiff ),
			dst( e, inDesc.BlobSize() );
		if( isMax ) {
			CIntBlob idx( e, outDesc.BlobSize() );
			CMaxPoolingDesc* desc = e.InitMaxPooling( inDesc, fh, fw, sh, sw, outDesc );
			const CIntHandle idxHandle = idx.Handle();
			try {
				e.BlobMaxPooling( *desc, src.Const(), &idxHandle, out.Handle() );
				e.BlobMaxPoolingBackward( *desc, grad.Const(), idx.Const(), dst.Handle() );
			} catch( ... ) {
				delete desc;
				throw;
			}
			delete desc;
		} else {
			CMeanPoolingDesc* desc = e.InitMeanPooling( inDesc, fh, fw, sh, sw, outDesc );
			try {
				e.BlobMeanPoolingBackward( *desc, grad.Const(), dst.Handle() );
			} catch( ... ) {
				delete desc;
				throw;
			}
			delete desc;
		}
		dst.CopyTo( sourceDiff );
	} );
}

SHIM_API int shim_blob_max_pooling( void* engine, const float* in, int n, int h, int w, int c, int fh, int fw,
	int sh, int sw, int* indices, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = ( h - fh ) / sh + 1, wo = ( w - fw ) / sw + 1;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), outDesc = imageDesc( n, ho, wo, c );
		CFloatBlob src( e, inDesc.BlobSize(), in ), dst( e, outDesc.BlobSize() );
		CIntBlob idx( e, outDesc.BlobSize() );
		CMaxPoolingDesc* desc = e.InitMaxPooling( inDesc, fh, fw, sh, sw, outDesc );
		const CIntHandle idxHandle = idx.Handle();
		try {
			e.BlobMaxPooling( *desc, src.Const(), indices != nullptr ? &idxHandle : nullptr, dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( out );
		if( indices != nullptr ) {
			idx.CopyTo( indices );
		}
	} );
}

SHIM_API int shim_blob_mean_pooling( void* engine, const float* in, int n, int h, int w, int c, int fh, int fw,
	int sh, int sw, float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int ho = ( h - fh ) / sh + 1, wo = ( w - fw ) / sw + 1;
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), outDesc = imageDesc( n, ho, wo, c );
		CFloatBlob src( e, inDesc.BlobSize(), in ), dst( e, outDesc.BlobSize() );
		CMeanPoolingDesc* desc = e.InitMeanPooling( inDesc, fh, fw, sh, sw, outDesc );
		try {
			e.BlobMeanPooling( *desc, src.Const(), dst.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		dst.CopyTo( out );
	} );
}

SHIM_API int shim_blob_resize_image( void* engine, const float* from, int n, int h, int w, int c, int dl, int dr,
	int dt, int db, int padding, float value, float* to )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const CBlobDesc inDesc = imageDesc( n, h, w, c ), outDesc = imageDesc( n, h + dt + db, w + dl + dr, c );
		CFloatBlob src( e, inDesc.BlobSize(), from ), dst( e, outDesc.BlobSize() );
		const TBlobResizePadding mode = padding == 0 ? TBlobResizePadding::Constant
			: ( padding == 1 ? TBlobResizePadding::Edge : TBlobResizePadding::Reflect );
		e.BlobResizeImage( inDesc, src.Handle(), dl, dr, dt, db, mode, value, outDesc, dst.Handle() );
		dst.CopyTo( to );
	} );
}

SHIM_API int shim_row_multiply_matrix_by_matrix( void* engine, const float* first, const float* second, int h, int w, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob a( e, h * w, first ), b( e, h * w, second ), out( e, h );
		e.RowMultiplyMatrixByMatrix( a.Const(), b.Const(), h, w, out.Handle() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_matrix_softmax_diff_op_by_rows( void* engine, const float* first, const float* second, int h, int w, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob a( e, h * w, first ), b( e, h * w, second ), out( e, h * w );
		e.MatrixSoftmaxDiffOpByRows( a.Const(), b.Const(), h, w, out.Handle() );
		out.CopyTo( result );
	} );
}

SHIM_API int shim_multiply_diag_matrix_by_matrix_and_add( void* engine, int batch, const float* first, int size, const float* second,
	int width, float* result )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob a( e, batch * size, first ), b( e, batch * size * width, second ), out( e, size * width, result );
		e.MultiplyDiagMatrixByMatrixAndAdd( batch, a.Const(), size, b.Const(), width, out.Handle() );
		out.CopyTo( result );
	} );
}

// InitDropout + Dropout (NeoMathEngine.h:930-935); dims: the 7 blob dimensions
SHIM_API int shim_dropout( void* engine, const int* dims, float rate, int isSpatial, int isBatchwise, int seed, const float* in,
	float* out )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CBlobDesc desc( CT_Float );
		for( int i = 0; i < 7; ++i ) {
			desc.SetDimSize( i, dims[i] );
		}
		CFloatBlob src( e, desc.BlobSize(), in ), dst( e, desc.BlobSize() );
		CDropoutDesc* dropout = e.InitDropout( rate, isSpatial != 0, isBatchwise != 0, desc, desc, seed );
		try {
			e.Dropout( *dropout, src.Handle(), dst.Handle() );
		} catch( ... ) {
			delete dropout;
			throw;
		}
		delete dropout;
		dst.CopyTo( out );
	} );
}

// BroadcastCopy (NeoMathEngine.h:75-83): toDims / fromDims are the 7 blob dimensions, without the additional width
SHIM_API int shim_broadcast_copy( void* engine, const int* toDims, const int* fromDims, int additionalWidth, const float* from,
	float* to )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CBlobDesc toDesc( CT_Float ), fromDesc( CT_Float );
		for( int i = 0; i < 7; ++i ) {
			toDesc.SetDimSize( i, toDims[i] );
			fromDesc.SetDimSize( i, fromDims[i] );
		}
		CFloatBlob src( e, fromDesc.BlobSize() * additionalWidth, from ), dst( e, toDesc.BlobSize() * additionalWidth );
		e.BroadcastCopy( dst.Handle(), src.Const(), toDesc, fromDesc, additionalWidth );
		dst.CopyTo( to );
	} );
}

// dims: [7] of the big blob; partDims: [count][7]; dim: the blob dimension to split / merge along
SHIM_API int shim_blob_split_merge( void* engine, int dim, const int* dims, float* big, const int* partDims,
	float* const* parts, int count, int merge )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CBlobDesc bigDesc( CT_Float );
		for( int i = 0; i < 7; ++i ) {
			bigDesc.SetDimSize( i, dims[i] );
		}
		std::vector<CBlobDesc> descs( count, CBlobDesc( CT_Float ) );
		std::vector<CFloatBlob*> blobs;
		std::vector<CFloatHandle> handles;
		for( int p = 0; p < count; ++p ) {
			for( int i = 0; i < 7; ++i ) {
				descs[p].SetDimSize( i, partDims[p * 7 + i] );
			}
			blobs.push_back( new CFloatBlob( e, descs[p].BlobSize(), merge ? parts[p] : nullptr ) );
			handles.push_back( blobs.back()->Handle() );
		}
		CFloatBlob bigBlob( e, bigDesc.BlobSize(), merge ? nullptr : big );
		try {
			if( merge ) {
				e.BlobMergeByDim( static_cast<TBlobDim>( dim ), descs.data(), handles.data(), count, bigDesc, bigBlob.Handle() );
				bigBlob.CopyTo( big );
			} else {
				e.BlobSplitByDim( static_cast<TBlobDim>( dim ), bigDesc, bigBlob.Const(), descs.data(), handles.data(), count );
				for( int p = 0; p < count; ++p ) {
					blobs[p]->CopyTo( parts[p] );
				}
			}
		} catch( ... ) {
			for( CFloatBlob* b : blobs ) delete b;
			throw;
		}
		for( CFloatBlob* b : blobs ) delete b;
	} );
}

SHIM_API int shim_lstm( void* engine, int H, int In, const float* wIn, const float* bIn, const float* wRec,
	const float* bRec, int reverse, int T, int B, const float* c0, const float* h0, const float* x, float* cOut, float* hOut )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob WIn( e, size_t( 4 ) * H * In, wIn ), WRec( e, size_t( 4 ) * H * H, wRec ), BIn( e, 4 * H, bIn ),
			BRec( e, 4 * H, bRec ), C0( e, size_t( B ) * H, c0 ), H0( e, size_t( B ) * H, h0 ), X( e, size_t( T ) * B * In, x ),
			COut( e, size_t( T ) * B * H ), HOut( e, size_t( T ) * B * H );
		CLstmDesc* desc = e.InitLstm( H, In, WIn.Const(), bIn != nullptr ? BIn.Const() : CConstFloatHandle(),
			WRec.Const(), bRec != nullptr ? BRec.Const() : CConstFloatHandle() );
		try {
			e.Lstm( *desc, reverse != 0, T, B, c0 != nullptr ? C0.Const() : CConstFloatHandle(),
				h0 != nullptr ? H0.Const() : CConstFloatHandle(), X.Const(),
				cOut != nullptr ? COut.Handle() : CFloatHandle(), HOut.Handle() );
		} catch( ... ) {
			delete desc;
			throw;
		}
		delete desc;
		HOut.CopyTo( hOut );
		if( cOut != nullptr ) {
			COut.CopyTo( cOut );
		}
	} );
}

// ---- memory interface of the engine (for the allocator behaviour tests) -----------------------------------

SHIM_API int shim_memory_stats( void* engine, size_t* peak, size_t* current, size_t* inPools )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		*peak = e.GetPeakMemoryUsage();
		*current = e.GetCurrentMemoryUsage();
		*inPools = e.GetMemoryInPools();
	} );
}

SHIM_API int shim_clean_up( void* engine )
{
	return guarded( [&]() { static_cast<IMathEngine*>( engine )->CleanUp(); } );
}

// IPerformanceCounters of the engine (PerformanceCounters.h:27-60), as CDnn::EnableProfile drives them: Synchronise(),
// work, Synchronise(), read. Two measurements, a small and a large element-wise pass; name64 receives counter 0's name.
SHIM_API int shim_performance_counters( void* engine, int smallSize, int largeSize, int repeats, char* name64, int* counterCount,
	unsigned long long* smallValue, unsigned long long* largeValue )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, largeSize ), out( e, largeSize );
		e.VectorFill( in.Handle(), 1.5f, largeSize );
		IPerformanceCounters* counters = e.CreatePerformanceCounters( true );
		if( counters == nullptr ) {
			throw std::runtime_error( "CreatePerformanceCounters returned null" );
		}
		*counterCount = static_cast<int>( counters->size() );
		std::strncpy( name64, ( *counters )[0].Name, 63 );
		name64[63] = 0;
		counters->Synchronise();
		// ( VectorExp: a call that an engine's stream launches at once; repeated calls of the kinds it may put aside
		// and run as one pass would not be `repeats` passes over memory )
		for( int i = 0; i < repeats; ++i ) {
			e.VectorExp( in.Const(), out.Handle(), smallSize );
		}
		counters->Synchronise();
		*smallValue = ( *counters )[0].Value;
		for( int i = 0; i < repeats; ++i ) {
			e.VectorExp( in.Const(), out.Handle(), largeSize );
		}
		counters->Synchronise();
		*largeValue = ( *counters )[0].Value;
		delete counters;
	} );
}

// probe for a method outside the implemented paths (asserts on engines that do not implement it, and on the reference CPU
// engine where it is built without MKL)
SHIM_API int shim_singular_value_decomposition( void* engine, const float* matrix, int height, int width, float* singular )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int rank = height < width ? height : width;
		CFloatBlob a( e, height * width, matrix ), u( e, height * rank ), sv( e, rank ), vt( e, rank * width ), superb( e, rank );
		e.SingularValueDecomposition( a.Handle(), height, width, u.Handle(), sv.Handle(), vt.Handle(), superb.Handle(), true, true );
		sv.CopyTo( singular );
	} );
}

// IMathEngine::CtcLossForward; label_lens, result_lens, weights and gradient may be null
SHIM_API int shim_ctc_loss_forward( void* engine, int result_len, int batch, int classes, int label_len, int blank, int skip_blanks,
	const float* result, const int* labels, const int* label_lens, const int* result_lens, const float* weights, float* loss,
	float* gradient )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		const int frames = result_len * batch * classes;
		CFloatBlob in( e, frames, result ), lossOut( e, 1 ), grad( e, frames ), w( e, batch );
		CIntHandleVar lab( e, label_len * batch + 1 ), labLens( e, batch ), resLens( e, batch );
		if( label_len > 0 ) {
			e.DataExchangeTyped<int>( lab.GetHandle(), labels, label_len * batch );
		}
		if( label_lens != nullptr ) {
			e.DataExchangeTyped<int>( labLens.GetHandle(), label_lens, batch );
		}
		if( result_lens != nullptr ) {
			e.DataExchangeTyped<int>( resLens.GetHandle(), result_lens, batch );
		}
		if( weights != nullptr ) {
			e.DataExchangeTyped<float>( w.Handle(), weights, batch );
		}
		e.CtcLossForward( result_len, batch, classes, label_len, blank, skip_blanks != 0, in.Const(), lab.GetHandle(),
			label_lens != nullptr ? CConstIntHandle( labLens.GetHandle() ) : CConstIntHandle(),
			result_lens != nullptr ? CConstIntHandle( resLens.GetHandle() ) : CConstIntHandle(),
			weights != nullptr ? w.Const() : CConstFloatHandle(), lossOut.Handle(), gradient != nullptr ? grad.Handle() : CFloatHandle() );
		lossOut.CopyTo( loss );
		if( gradient != nullptr ) {
			grad.CopyTo( gradient );
		}
	} );
}

SHIM_API int shim_vector_top_k( void* engine, const float* first, int n, int k, float* result, int* indices )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, n, first ), out( e, k );
		CIntHandleVar found( e, k );
		e.VectorTopK( in.Const(), n, k, out.Handle(), found.GetHandle() );
		out.CopyTo( result );
		e.DataExchangeTyped<int>( indices, found.GetHandle(), k );
	} );
}

SHIM_API int shim_vector_power( void* engine, float exponent, const float* first, float* result, int n )
{
	return guarded( [&]() {
		IMathEngine& e = *static_cast<IMathEngine*>( engine );
		CFloatBlob in( e, n, first ), out( e, n );
		e.VectorPower( exponent, in.Const(), out.Handle(), n );
		out.CopyTo( result );
	} );
}
