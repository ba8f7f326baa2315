#include "HipLstmLayer.h"

namespace NeoML {

REGISTER_NEOML_LAYER( CHipLstmLayer, "NeoMLHipLstmLayer" )

CHipLstmLayer::CHipLstmLayer( IMathEngine& mathEngine ) :
	CLstmLayer( mathEngine ),
	fusedDesc( nullptr ),
	lastRunFused( false )
{
}

CHipLstmLayer::~CHipLstmLayer()
{
	InvalidateFusedWeights();
}

void CHipLstmLayer::InvalidateFusedWeights()
{
	delete fusedDesc;
	fusedDesc = nullptr;
	inputWeights = nullptr;
	inputFreeTerm = nullptr;
	recurWeights = nullptr;
	recurFreeTerm = nullptr;
}

void CHipLstmLayer::Reshape()
{
	CLstmLayer::Reshape();
	InvalidateFusedWeights();
}

void CHipLstmLayer::RunOnce()
{
	// the reference's conditions for the fused call (LstmLayer.cpp:352-356) without the engine-type test; on the CPU
	// engine the base class already does the same thing
	const bool fused = MathEngine().GetType() != MET_Cpu && !IsInCompatibilityMode() && !IsBackwardPerformed()
		&& !IsLearningPerformed() && GetRecurrentActivation() == AF_Sigmoid;
	lastRunFused = fused;
	if( !fused ) {
		CLstmLayer::RunOnce();
		return;
	}
	if( fusedDesc == nullptr ) {
		inputWeights = GetInputWeightsData();
		inputFreeTerm = GetInputFreeTermData();
		recurWeights = GetRecurWeightsData();
		recurFreeTerm = GetRecurFreeTermData();
		NeoAssert( inputWeights != nullptr && recurWeights != nullptr );
		fusedDesc = MathEngine().InitLstm( GetHiddenSize(), inputBlobs[0]->GetObjectSize(), inputWeights->GetData(),
			inputFreeTerm == nullptr ? CConstFloatHandle() : inputFreeTerm->GetData(), recurWeights->GetData(),
			recurFreeTerm == nullptr ? CConstFloatHandle() : recurFreeTerm->GetData() );
	}
	// inputs 1 and 2 are the optional initial state and output, output 1 the optional state sequence
	// (LstmLayer.cpp:358-364)
	const CConstFloatHandle inputStateBackLink = inputBlobs.Size() > 1 ? inputBlobs[1]->GetData() : CConstFloatHandle();
	const CConstFloatHandle inputMainBackLink = inputBlobs.Size() > 2 ? inputBlobs[2]->GetData() : CConstFloatHandle();
	const CFloatHandle outputState = outputBlobs.Size() > 1 ? outputBlobs[1]->GetData() : CFloatHandle();
	MathEngine().Lstm( *fusedDesc, IsReverseSequence(), inputBlobs[0]->GetBatchLength(), inputBlobs[0]->GetBatchWidth(),
		inputStateBackLink, inputMainBackLink, inputBlobs[0]->GetData(), outputState, outputBlobs[0]->GetData() );
}

} // namespace NeoML
