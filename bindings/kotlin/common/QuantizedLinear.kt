// Linear over a quantized weight (core/src/commonMain/kotlin/sk/ai/net/nn/Linear.kt:22-50).  The reference's Linear
// needs no change at all when it is constructed with initWeights = a QuantizedTensor and initBias = a DeviceTensor and
// fed DeviceTensor inputs: its forward is input.matmul(weight.t()) + bias, and both calls dispatch to the device
// (DeviceTensor.matmul / DeviceTensor.plus).  This module is the same thing without the zero-filled default tensors.
package sk.ai.net.hip

import sk.ai.net.Tensor
import sk.ai.net.nn.Module
import sk.ai.net.nn.reflection.ModuleParameter
import sk.ai.net.nn.reflection.ModuleParameters
import sk.ai.net.nn.reflection.bias
import sk.ai.net.nn.reflection.weights

class QuantizedLinear(
    weight: QuantizedTensor,
    bias: DeviceTensor? = null,
    override val name: String = "Linear",
) : Module(), ModuleParameters {

    override val params: List<ModuleParameter> = buildList {
        add(ModuleParameter.WeightParameter("$name.weight", weight))
        if (bias != null) add(ModuleParameter.BiasParameter("$name.bias", bias))
    }

    override val modules: List<Module> get() = emptyList()

    override fun forward(input: Tensor): Tensor {
        val x = if (input is DeviceTensor) input else DeviceTensor.of((params.weights().value as QuantizedTensor).ctx, hostAsDoubles(input))
        val y = x.matmul(params.weights().value.t())
        return if (params.size > 1) y + params.bias().value else y
    }

    private fun hostAsDoubles(t: Tensor) = t as? sk.ai.net.impl.DoublesTensor
        ?: throw IllegalArgumentException("QuantizedLinear takes DeviceTensor or DoublesTensor inputs")
}
