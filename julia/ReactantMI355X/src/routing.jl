# The bindings of src/mlir/libMLIR_h.jl that the non-sharded PJRT path calls, redefined to pick the
# library by the owner of one handle argument.  Every row: name, return type, (argument, C type)...,
# and which argument decides.  Types are those of the reference's bindings (all opaque handle types
# are `Cvoid` there) and of include/reactant_mi355x.h.
#
# Callers (reference): src/xla/PJRT/Client.jl:12-88, Device.jl:5-48, Buffer.jl:9-17,20-161,
# Future.jl:10-28, LoadedExecutable.jl:15-60; src/ConcreteRArray.jl (CopyToBuffer / CopyFromBuffer).

const P = Ptr{Cvoid}

const ROUTED = [
    # --- client / device
    (:FreeClient, Cvoid, [(:client, P)], 1),
    (:ClientNumDevices, Cint, [(:client, P)], 1),
    (:ClientNumAddressableDevices, Cint, [(:client, P)], 1),
    (:ClientProcessIndex, Cint, [(:client, P)], 1),
    (:ClientGetDevice, P, [(:client, P), (:device_id, Cint)], 1),
    (:ClientGetAddressableDevice, P, [(:client, P), (:device_id, Cint)], 1),
    (:ClientGetPlatformName, Cstring, [(:client, P)], 1),
    (:ClientGetDevices, Cvoid, [(:client, P), (:out_devices, Ptr{P})], 1),
    (:ClientGetAddressableDevices, Cvoid, [(:client, P), (:out_devices, Ptr{P})], 1),
    (:DeviceGetKind, Cstring, [(:device, P)], 1),
    (:DeviceToClient, P, [(:device, P)], 1),
    (:PjRtDeviceGetLocalDeviceId, Int64, [(:device, P)], 1),
    (:PjRtDeviceGetLocalHardwareId, Int64, [(:device, P)], 1),
    (:pjrt_device_is_addressable, Bool, [(:device, P)], 1),
    (:PjRtDeviceGetAllocatorStats, Cvoid, [(:device, P), (:jlstats, Ptr{API.JLAllocatorStats})], 1),
    # --- buffers
    (:ArrayFromHostBuffer, P, [(:client, P), (:data, P), (:ptype, UInt64), (:dim, Csize_t), (:cshape, Ptr{Int64}), (:device, P)], 1),
    (:UninitPJRTBuffer, P, [(:client, P), (:device, P), (:ptype, UInt64), (:shapeLen, UInt64), (:shape, Ptr{UInt64})], 1),
    (:BufferToHost, Cvoid, [(:buffer, P), (:data, P)], 1),
    (:CopyToBuffer, Cvoid, [(:client, P), (:buffer, P), (:data, P), (:offset, Csize_t), (:size, Csize_t), (:bufferP, Ptr{P})], 2),
    (:CopyFromBuffer, Cvoid, [(:client, P), (:buffer, P), (:data, P), (:offset, Csize_t), (:size, Csize_t), (:bufferP, Ptr{P})], 2),
    (:BufferShape, Ptr{Int64}, [(:buffer, P)], 1),
    (:BufferNDimensions, Int64, [(:buffer, P)], 1),
    (:BufferPrimitiveType, Cint, [(:buffer, P)], 1),
    (:BufferToDevice, P, [(:buffer, P)], 1),
    (:BufferToClient, P, [(:buffer, P)], 1),
    (:BufferOnCPU, UInt8, [(:buffer, P)], 1),
    (:UnsafeBufferPointer, P, [(:buffer, P)], 1),
    (:CopyBufferToDevice, P, [(:buffer, P), (:dst_device, P)], 1),
    (:PjRtBufferFree, Cvoid, [(:buffer, P)], 1),
    # --- futures
    (:FreeFuture, Cvoid, [(:future, P)], 1),
    (:FutureIsReady, UInt8, [(:future, P)], 1),
    (:FutureAwait, Cvoid, [(:future, P)], 1),
    # --- executables
    (:ExecutableFree, Cvoid, [(:exec, P)], 1),
    (:PjRtLoadedExecutableGetClient, P, [(:exec, P)], 1),
    (:PjRtLoadedExecutableGetHloModules, Cvoid, [(:exec, P), (:hlo_modules, Ptr{P}), (:nmodules, Ptr{Int32})], 1),
    (:XLAExecuteSharded, Cvoid,
     [(:exec, P), (:num_args, Cint), (:op_args, Ptr{P}), (:device, P), (:is_arg_donatable, Ptr{UInt8}), (:num_results, Cint),
      (:op_results, Ptr{P}), (:futures, Ptr{UInt8}), (:future_results, Ptr{P})], 1),
]

# `ccall` converts every argument with `Base.cconvert` / `unsafe_convert` to the declared type, exactly as
# the `@ccall` of the reference binding does, so callers that pass `Ref{NTuple{N,Ptr{Cvoid}}}`, arrays or
# `RefValue`s keep working.  A handle argument may arrive as a `Ptr`; ownership is asked with the raw
# address.
function route_definition(name::Symbol, ret, args, key::Int)
    names = [a[1] for a in args]
    types = Expr(:tuple, [a[2] for a in args]...)
    handle = names[key]
    lib_call = Expr(:call, :ccall, Expr(:tuple, QuoteNode(name), :mlir_c), ret, types, names...)
    own_call = Expr(:call, :ccall, :($(sym)($(QuoteNode(name)))), ret, types, names...)
    return quote
        function $name($(names...))
            if $(owns)($handle isa Ptr ? $handle : Base.unsafe_convert($(P), Base.cconvert($(P), $handle)))
                return $own_call
            end
            return $lib_call
        end
    end
end

function install_routes!()
    for (name, ret, args, key) in ROUTED
        Core.eval(API, route_definition(name, ret, args, key))
    end
    return nothing
end
