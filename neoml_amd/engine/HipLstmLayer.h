// CHipLstmLayer: NeoML's LSTM layer with the engine's fused IMathEngine::Lstm reached on a non-CPU engine.
//
// CLstmLayer::RunOnce only takes the fused path when GetType() == MET_Cpu
// (NeoML/src/Dnn/Layers/LstmLayer.cpp:350-370); on every other engine it unrolls the composite per-step graph
// (two fully connected layers, split, four activations, products and sums: some 15 launches per time step).
// This subclass is the opt-in way around that test for inference: same parameters, same serialization, same
// inputs and outputs as CLstmLayer, and the same conditions for the fused path except the engine type. Whenever a
// condition does not hold (learning, backward, compatibility mode, another recurrent activation) it behaves exactly
// as its base class.
//
// The fused call needs the weights as engine handles; CLstmLayer keeps them private to its inner layers, so the layer
// takes copies through the public accessors the first time it runs after a Reshape. Weights set through
// Set*WeightsData / Set*FreeTermData afterwards are picked up by calling InvalidateFusedWeights() (or any Reshape).
#pragma once

#include <NeoML/NeoML.h>

namespace NeoML {

class __attribute__( ( visibility( "default" ) ) ) CHipLstmLayer : public CLstmLayer {
	NEOML_DNN_LAYER( CHipLstmLayer )
public:
	explicit CHipLstmLayer( IMathEngine& mathEngine );
	~CHipLstmLayer() override;

	void RunOnce() override;
	void Reshape() override;

	// Drops the weight copies and the engine descriptor; the next RunOnce takes fresh ones.
	void InvalidateFusedWeights();

	// true when the last RunOnce went through IMathEngine::Lstm
	bool LastRunWasFused() const { return lastRunFused; }

private:
	CLstmDesc* fusedDesc;
	CPtr<CDnnBlob> inputWeights, inputFreeTerm, recurWeights, recurFreeTerm;
	bool lastRunFused;
};

} // namespace NeoML
