# Compilation: the optimized module goes over as text.
#
# Reference: `XLA.compile(client::PJRT.Client, mod::MLIR.IR.Module; ...)`
# (src/xla/PJRT/LoadedExecutable.jl:62-83) calls the hand-written binding
# `MLIR.API.ClientCompileWithProto(client, mod, bytes, length)` (src/mlir/MLIR.jl:61-71,
# deps/ReactantExtra/API.cpp:1528-1536), then wraps the handle with the counts the caller supplies.
# Only that binding is redefined: for a client of this library it prints the module
# (`string(mod)`, the call Compiler.jl uses for its own dumps) and calls ClientCompileFromText;
# the compile-options proto is passed along and ignored there (one device, no sharding).
# `XLA.get_hlo_modules`, called after every compile, goes through the routed
# PjRtLoadedExecutableGetHloModules, which reports zero modules for these executables.

function compile_text(client::Ptr{Cvoid}, text::String, options::Vector{UInt8})
    GC.@preserve text options begin
        exec = ccall(
            sym(:ClientCompileFromText),
            Ptr{Cvoid},
            (Ptr{Cvoid}, Ptr{UInt8}, Csize_t, Ptr{UInt8}, Csize_t),
            client,
            pointer(text),
            sizeof(text),
            isempty(options) ? Ptr{UInt8}(C_NULL) : pointer(options),
            length(options),
        )
    end
    return exec
end

function install_compile!()
    Core.eval(
        API,
        quote
            function ClientCompileWithProto(
                client, cmod, compile_options_proto::Vector{UInt8}, compile_options_proto_size
            )
                if $(owns)(client)
                    return $(compile_text)(client, string(cmod), compile_options_proto)
                end
                return ccall(
                    (:ClientCompileWithProto, mlir_c),
                    Ptr{PjRtLoadedExecutable},
                    (Ptr{PjRtClient}, MlirModule, Ptr{UInt8}, Csize_t),
                    client,
                    cmod,
                    compile_options_proto,
                    compile_options_proto_size,
                )
            end
        end,
    )
    install_device_properties!()
    return nothing
end
