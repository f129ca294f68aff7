classdef BatchNormalizationLayer < BatchNormalizationLayer & nnvhip.RowMapLayer
    % BatchNormalizationLayer whose star reach (BatchNormalizationLayer.m:247-351, 384-413) runs on
    % the device, with the reference's order of operations.
    methods
        function obj = BatchNormalizationLayer(varargin)
            obj = obj@BatchNormalizationLayer(varargin{:});
        end
        function [ops, scopes, params] = row_program(obj, h, w, c, isImage)
            ops = []; scopes = []; params = [];
            if isempty(obj.TrainedMean) || isempty(obj.TrainedVariance) || isempty(obj.Epsilon) || isempty(obj.Offset) || isempty(obj.Scale)
                return;
            end
            pr = @(a) nnvhip.RowMapLayer.per_row(a, h, w, c);
            if isImage   % :286-330: c - mean; all ./ sqrt(var + eps); all .* scale; c + offset
                ops = [1 3 2 0]; scopes = [0 1 1 0];
                params = [pr(obj.TrainedMean), pr(sqrt(obj.TrainedVariance(:) + obj.Epsilon)), pr(obj.Scale), pr(obj.Offset)];
            else         % :332-349: l = scale ./ sqrt(var + eps); b = offset - mean .* l
                l = obj.Scale(:) ./ sqrt(obj.TrainedVariance(:) + obj.Epsilon);
                b = obj.Offset(:) - obj.TrainedMean(:) .* l;
                ops = [2 0]; scopes = [1 0];
                params = [pr(l), pr(b)];
            end
        end
        function images = reach_star_multipleInputs(obj, in_images, option) %#ok<INUSD>
            for i = 1:length(in_images)
                if ~isa(in_images(i), 'ImageStar') && ~isa(in_images(i), 'Star')
                    error('Input is not a Star, ImageStar or VolumeStar');
                end
            end
            images = obj.apply_rowmap(in_images);
        end
        function image = reach_star_single_input(obj, in_image)
            image = obj.reach_star_multipleInputs(in_image, 'single');
        end
    end
end
